// Causal attention over the paged key/value cache: the kernel that takes every
// shape (any head counts and groups, head sizes in steps of 8 up to 256, any page
// size that is a multiple of 8, a window or none), for 32-bit and bfloat16 storage.
//
// One wave per (token, head).  A token's request, its absolute position p and the
// keys it sees, [lo, p] with lo = max(0, p - window + 1) (0 without a window), come
// from the batch arrays.  Keys are walked in chunks of 64 that start at multiples of
// 64, a lane per key; scores, the running maximum and sum (online softmax) and the
// output are 32-bit.  What a (token, head) computes, and the order it adds in,
// depends on p and the cache's contents only: not on how the step's tokens were cut,
// not on other requests in the batch, not on which pages hold the keys.
//
// head_slopes (may be null): a bias inside the scores that grows with the distance, for position
// encodings of that kind: slope[h] * (j - p) is added to the scaled score of key j for the query at p.
#include "common.h"
#include "kv_layout.h"

constexpr int MAX_HEAD_DIM = 256;

template <class T>
__global__ void __launch_bounds__(64)
paged_attention_generic_kernel(const T *__restrict__ q, int q_stride, T *__restrict__ out, int out_stride,
                               const T *__restrict__ cache, const int *__restrict__ block_table, int max_pages,
                               const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                               const int *__restrict__ req_of_token, int nh, int nkvh, int dh, int page,
                               float scale, int window, const float *__restrict__ head_slopes) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int r = req_of_token[t];
    const int p = ctx_len[r] - (q_start[r + 1] - t);
    const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
    const int kvh = h / (nh / nkvh);
    const int dh8 = dh / 8;
    const float slope = head_slopes ? head_slopes[h] : 0.f;
    __shared__ float qs[MAX_HEAD_DIM];
    __shared__ float ps[WAVE];
    for (int c = lane; c < dh; c += WAVE) qs[c] = to_f32(q[(size_t)t * q_stride + (size_t)h * dh + c]);
    __syncthreads();

    const int *bt = block_table + (size_t)r * max_pages;
    const size_t page_elems = kv_page_elems(nkvh, dh, page);
    const size_t v_base = (size_t)nkvh * dh * page + (size_t)kvh * dh * page;
    float m = -INFINITY, l = 0.f;
    float o[MAX_HEAD_DIM / WAVE] = {0.f, 0.f, 0.f, 0.f};

    for (int base = (lo / WAVE) * WAVE; base <= p; base += WAVE) {
        const int j = base + lane;
        const bool valid = j >= lo && j <= p;
        float s = -INFINITY;
        if (valid) {
            const int pg = bt[j / page], tok = j % page;
            const T *kp = cache + (size_t)pg * page_elems + ((size_t)kvh * dh8 * page + tok) * 8;
            float acc = 0.f;
            for (int c8 = 0; c8 < dh8; ++c8) {
                const T *kk = kp + (size_t)c8 * page * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc += qs[c8 * 8 + e] * to_f32(kk[e]);
            }
            s = acc * scale + slope * (float)(j - p);
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float pj = valid ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);      // 0 in the first chunk (m = -inf)
        l = l * alpha + wave_sum(pj);
        m = m_new;
        ps[lane] = pj;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MAX_HEAD_DIM / WAVE; ++i) o[i] *= alpha;
        const int j_first = base > lo ? base : lo;
        const int j_last = base + WAVE - 1 < p ? base + WAVE - 1 : p;
        for (int j2 = j_first; j2 <= j_last; ++j2) {
            const float pp = ps[j2 - base];
            const int pg = bt[j2 / page], tok = j2 % page;
            const T *vp = cache + (size_t)pg * page_elems + v_base + tok;
#pragma unroll
            for (int i = 0; i < MAX_HEAD_DIM / WAVE; ++i) {
                const int d = lane + WAVE * i;
                if (d < dh) o[i] += pp * to_f32(vp[(size_t)d * page]);
            }
        }
        __syncthreads();
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < MAX_HEAD_DIM / WAVE; ++i) {
        const int d = lane + WAVE * i;
        if (d < dh) out[(size_t)t * out_stride + (size_t)h * dh + d] = from_f32<T>(o[i] * inv);
    }
}

// q: [n, q_stride] (head h of token t at t*q_stride + h*dh), out: [n, out_stride].
// cache: one layer's pages.  block_table: [n_req, max_pages] page ids (an entry that a
// window has passed may hold anything: it is not read).  q_start: [n_req + 1] offsets of
// the requests' tokens in the batch, ctx_len: [n_req] tokens each request holds after
// this step, req_of_token: [n].  head_slopes: null or [nh] 32-bit.
LCU_API int lcu_paged_attention_generic(const void *q, int q_stride, void *out, int out_stride, int type,
                                        const void *cache, const int *block_table, int max_pages,
                                        const int *q_start, const int *ctx_len, const int *req_of_token, int n,
                                        int nh, int nkvh, int dh, int page, float scale, int window,
                                        const float *head_slopes, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || dh <= 0 || dh % 8 || dh > MAX_HEAD_DIM || page <= 0 || page % 8 ||
        max_pages <= 0 || window < 0 || nh > 65535)
        return LCU_BAD_ARGUMENT;
    dim3 grid(n, nh), block(WAVE);
    if (type == LCU_F32)
        paged_attention_generic_kernel<float><<<grid, block, 0, stream>>>((const float *)q, q_stride, (float *)out, out_stride, (const float *)cache, block_table, max_pages, q_start, ctx_len, req_of_token, nh, nkvh, dh, page, scale, window, head_slopes);
    else if (type == LCU_BF16)
        paged_attention_generic_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t *)q, q_stride, (bf16_t *)out, out_stride, (const bf16_t *)cache, block_table, max_pages, q_start, ctx_len, req_of_token, nh, nkvh, dh, page, scale, window, head_slopes);
    else
        return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
