// Plain C++ references of the kernels: contiguous loops over float32 arrays, sums in 64-bit,
// no tiling, no paging tricks.  Each kernel of csrc/kernels is tested against the function
// here that computes the same thing, and these are tested against the plain Python
// implementation; they share no code with the kernels (the page layout is written out again
// below).  Formulas follow the reference (YdrMaster/llama.cu); paths are relative to its root.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <vector>

#define API extern "C" __attribute__((visibility("default")))

namespace ref {

// out[i, :] = table[ids[i], :]            llama.cu/src/op/embedding.cuh:6-8
void embedding(const float *table, const int *ids, int n, int d, float *out) {
    for (int i = 0; i < n; ++i)
        for (int c = 0; c < d; ++c) out[(size_t)i * d + c] = table[(size_t)ids[i] * d + c];
}

// y = x * rsqrt(sum(x^2) / d + eps) * w    llama.cu/src/op/rms_norm.cuh:15-29
void rms_norm(const float *x, const float *w, float eps, int n, int d, float *y) {
    for (int i = 0; i < n; ++i) {
        const float *row = x + (size_t)i * d;
        double acc = 0;
        for (int c = 0; c < d; ++c) acc += (double)row[c] * row[c];
        const double rms = 1.0 / std::sqrt(acc / d + (double)eps);
        for (int c = 0; c < d; ++c) y[(size_t)i * d + c] = (float)(rms * row[c] * w[c]);
    }
}

// out[m, n] = sum_k a[m, k] * w[n, k]     the weight is stored [out, in]: llama.cu/src/op/linear.rs:85-89
void gemm_nt(const float *a, const float *w, int m, int n, int k, float *out) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double acc = 0;
            for (int c = 0; c < k; ++c) acc += (double)a[(size_t)i * k + c] * w[(size_t)j * k + c];
            out[(size_t)i * n + j] = (float)acc;
        }
}

// out = gate * sigmoid(gate) * up for gate_up = [gate | up]      llama.cu/src/op/swiglu.cuh:1-3,17-19
void swiglu(const float *gate_up, int n, int di, float *out) {
    for (int i = 0; i < n; ++i)
        for (int c = 0; c < di; ++c) {
            const double g = gate_up[(size_t)i * 2 * di + c], u = gate_up[(size_t)i * 2 * di + di + c];
            out[(size_t)i * di + c] = (float)(g * (1.0 / (1.0 + std::exp(-g))) * u);
        }
}

// One page of a layer's cache: first all keys, [kv_head][dim / 8][token][8], then all values,
// [kv_head][dim][token].
static size_t page_elems(int nkvh, int dh, int page) { return (size_t)2 * nkvh * dh * page; }
static size_t key_at(int kvh, int tok, int dim, int dh, int page) {
    return (((size_t)kvh * (dh / 8) + dim / 8) * page + tok) * 8 + dim % 8;
}
static size_t value_at(int nkvh, int kvh, int tok, int dim, int dh, int page) {
    return (size_t)nkvh * dh * page + ((size_t)kvh * dh + dim) * page + tok;
}

// The rotation tables as llama.cu/src/model/mod.rs:200-209 makes them: in 32-bit,
// freq_i = theta^(-(2 i / rot_dim)), angle = pos * freq_i; sine and cosine of that 32-bit angle.
static void angle(int pos, int i, int rot_dim, float theta, double &s, double &c) {
    const float expo = -((2.0f * (float)i) / (float)rot_dim);
    const float freq = std::pow(theta, expo);
    const float ang = (float)pos * freq;
    s = std::sin((double)ang);
    c = std::cos((double)ang);
}

// Rotate q (in place) and k of every token by its position, (a, b) -> (a cos - b sin, a sin + b cos)
// (llama.cu/src/op/rope.cuh:26-34; pairing 1 pairs neighbours (2i, 2i+1) as there, pairing 0 pairs
// (i, i + rot_dim / 2)), and write the rotated keys and the values into the token's place in the
// pages: slots[t] = page * page_size + place, or -1 to store nothing.  qkv: [n, (nh + 2 nkvh) * dh].
void rope_kv_write(float *qkv, int n, const int *positions, const int *slots, float theta, int nh, int nkvh, int dh,
                   int rot_dim, int pairing, int page, float *cache) {
    const int width = (nh + 2 * nkvh) * dh, half = rot_dim / 2;
    for (int t = 0; t < n; ++t) {
        float *row = qkv + (size_t)t * width;
        for (int h = 0; h < nh + nkvh; ++h) {
            float *x = row + (size_t)h * dh;
            for (int i = 0; i < half; ++i) {
                const int ia = pairing ? 2 * i : i, ib = pairing ? 2 * i + 1 : i + half;
                double s, c;
                angle(positions[t], i, rot_dim, theta, s, c);
                const double a = x[ia], b = x[ib];
                x[ia] = (float)(a * c - b * s);
                x[ib] = (float)(a * s + b * c);
            }
        }
        if (!cache || slots[t] < 0) continue;
        float *pg = cache + (size_t)(slots[t] / page) * page_elems(nkvh, dh, page);
        const int place = slots[t] % page;
        for (int h = 0; h < nkvh; ++h)
            for (int c = 0; c < dh; ++c) {
                pg[key_at(h, place, c, dh, page)] = row[(size_t)(nh + h) * dh + c];
                pg[value_at(nkvh, h, place, c, dh, page)] = row[(size_t)(nh + nkvh + h) * dh + c];
            }
    }
}

// Causal attention of the step's queries over the pages (the call contract of
// llama.cu/src/exec/step.rs:162-178: causal, offset by the request's position).  Request r feeds
// the tokens q_start[r] .. q_start[r + 1] - 1, which stand at the positions ctx_len[r] - count ..
// ctx_len[r] - 1; the query at position p sees the keys max(0, p - window + 1) .. p (window 0: all
// from 0); head h reads key/value head h / (nh / nkvh); key j lies in page block_table[r][j / page].
void paged_attention(const float *q, int q_stride, const float *cache, const int *block_table, int max_pages,
                     const int *q_start, const int *ctx_len, int n_req, int nh, int nkvh, int dh, int page, float scale,
                     int window, float *out) {
    const int g = nh / nkvh;
    std::vector<double> s;
    for (int r = 0; r < n_req; ++r) {
        const int count = q_start[r + 1] - q_start[r];
        for (int i = 0; i < count; ++i) {
            const int t = q_start[r] + i, p = ctx_len[r] - count + i;
            const int lo = window > 0 ? std::max(0, p - window + 1) : 0;
            for (int h = 0; h < nh; ++h) {
                const float *qh = q + (size_t)t * q_stride + (size_t)h * dh;
                const int kvh = h / g;
                s.assign(p - lo + 1, 0.0);
                double mx = -INFINITY;
                for (int j = lo; j <= p; ++j) {
                    const float *pg = cache + (size_t)block_table[(size_t)r * max_pages + j / page] * page_elems(nkvh, dh, page);
                    double acc = 0;
                    for (int c = 0; c < dh; ++c) acc += (double)qh[c] * pg[key_at(kvh, j % page, c, dh, page)];
                    s[j - lo] = acc * scale;
                    mx = std::max(mx, s[j - lo]);
                }
                double sum = 0;
                for (double &v : s) { v = std::exp(v - mx); sum += v; }
                for (int c = 0; c < dh; ++c) {
                    double acc = 0;
                    for (int j = lo; j <= p; ++j) {
                        const float *pg = cache + (size_t)block_table[(size_t)r * max_pages + j / page] * page_elems(nkvh, dh, page);
                        acc += s[j - lo] * pg[value_at(nkvh, kvh, j % page, c, dh, page)];
                    }
                    out[(size_t)t * nh * dh + (size_t)h * dh + c] = (float)(acc / sum);
                }
            }
        }
    }
}

// One token from one row of logits.  Greedy (temperature 0 or top_k 1,
// llama.cu/src/op/random_sample/mod.rs:80-82): the largest logit, the lowest index among equals.
// Otherwise llama.cu/src/op/random_sample/sample.cuh:186-207 and :71-87: sort descending (stable),
// w_0 = 1, w_i = exp((l_i - l_0) / T), inclusive prefix sums c, p = u * min(top_p * c[n-1],
// c[top_k - 1]), the first i with c[i] >= p; the answer is that entry's index before sorting.
int sample(const float *logits, int n, float temperature, float top_p, long long top_k, float u) {
    if (temperature == 0.f || top_k == 1) {
        int best = 0;
        for (int i = 1; i < n; ++i)
            if (logits[i] > logits[best]) best = i;
        return best;
    }
    std::vector<int> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return logits[a] > logits[b]; });
    std::vector<double> c(n);
    double run = 0;
    for (int i = 0; i < n; ++i) {
        run += i == 0 ? 1.0 : std::exp(((double)logits[order[i]] - (double)logits[order[0]]) / (double)temperature);
        c[i] = run;
    }
    const long long k = std::min<long long>(top_k, n);
    const double p = (double)u * std::min((double)top_p * c[n - 1], c[k - 1]);
    for (int i = 0; i < n; ++i)
        if (c[i] >= p) return order[i];
    return order[n - 1];
}

}  // namespace ref

API void lcu_ref_embedding(const float *table, const int *ids, int n, int d, float *out) { ref::embedding(table, ids, n, d, out); }
API void lcu_ref_rms_norm(const float *x, const float *w, float eps, int n, int d, float *y) { ref::rms_norm(x, w, eps, n, d, y); }
API void lcu_ref_gemm_nt(const float *a, const float *w, int m, int n, int k, float *out) { ref::gemm_nt(a, w, m, n, k, out); }
API void lcu_ref_swiglu(const float *gate_up, int n, int di, float *out) { ref::swiglu(gate_up, n, di, out); }
API void lcu_ref_rope_kv_write(float *qkv, int n, const int *positions, const int *slots, float theta, int nh, int nkvh, int dh,
                               int rot_dim, int pairing, int page, float *cache) {
    ref::rope_kv_write(qkv, n, positions, slots, theta, nh, nkvh, dh, rot_dim, pairing, page, cache);
}
API void lcu_ref_paged_attention(const float *q, int q_stride, const float *cache, const int *block_table, int max_pages,
                                 const int *q_start, const int *ctx_len, int n_req, int nh, int nkvh, int dh, int page,
                                 float scale, int window, float *out) {
    ref::paged_attention(q, q_stride, cache, block_table, max_pages, q_start, ctx_len, n_req, nh, nkvh, dh, page, scale, window, out);
}
API int lcu_ref_sample(const float *logits, int n, float temperature, float top_p, long long top_k, float u) {
    return ref::sample(logits, n, temperature, top_p, top_k, u);
}
