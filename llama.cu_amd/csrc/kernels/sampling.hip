// Sampling from rows of float32 logits: arg-max, and temperature sampling with
// top-k and top-p cuts.
//
// The reference sorts a row descending, sets w_0 = 1 and w_i = exp((l_i - l_0)/T),
// takes inclusive prefix sums c, draws p = u * min(top_p * c[n-1], c[top_k-1]) and
// returns the first entry with c[i] >= p (llama.cu/src/op/random_sample/sample.cuh:71-87,
// 186-207, with library sort, scan and reduce).  The same token comes out here without
// sorting: the entry with c[i] >= p is found by a radix select over the bit patterns of
// the logits, most significant byte first, on histograms of counts and of weights.
// Weights are summed as 64-bit fixed-point integers (w * 2^45), so the sums do not
// depend on the order of the additions and a draw is reproducible bit for bit.  Equal
// logits are ordered by index, as a stable sort orders them.
#include "common.h"

constexpr int SAMPLE_THREADS = 1024;
constexpr double FIXED_ONE = 35184372088832.0;   // 2^45: the sum of 2^19 weights of 1 still fits 64 bits
constexpr int MAX_VOCAB = 1 << 19;

__device__ __forceinline__ uint32_t order_key(float x) {
    // ascending float order -> ascending unsigned order
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ unsigned long long fixed_weight(float logit, float max_logit, float inv_t) {
    const float w = expf((logit - max_logit) * inv_t);
    return (unsigned long long)((double)w * FIXED_ONE);
}

// ---------------------------------------------------------------- arg-max
// The largest logit of each row; among equals the lowest index.  NaN never wins.
__global__ void __launch_bounds__(SAMPLE_THREADS)
argmax_kernel(const float *__restrict__ logits, int ld, int vocab, int *__restrict__ out) {
    const float *row = logits + (size_t)blockIdx.x * ld;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    // four neighbouring logits per load where the row allows it (many loads in flight: a
    // row is read by one workgroup, so latency, not bandwidth, is what counts)
    const int vec_end = (((size_t)row % 16) == 0) ? (vocab / 4) * 4 : 0;
#pragma unroll 4
    for (int i = threadIdx.x * 4; i < vec_end; i += blockDim.x * 4) {
        const float4 v = *(const float4 *)(row + i);
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (e[k] > best || (e[k] == best && i + k < bi)) { best = e[k]; bi = i + k; }
    }
    for (int i = vec_end + threadIdx.x; i < vocab; i += blockDim.x) {
        const float v = row[i];
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    }
    __shared__ float sv[SAMPLE_THREADS / WAVE];
    __shared__ int si[SAMPLE_THREADS / WAVE];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, WAVE);
        const int oi = __shfl_xor(bi, off, WAVE);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    if (lane == 0) { sv[wave] = best; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x / WAVE); ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

LCU_API int lcu_argmax(const float *logits, int ld, int rows, int vocab, int *out, hipStream_t stream) {
    if (rows <= 0) return LCU_OK;
    if (vocab <= 0 || ld < vocab) return LCU_BAD_ARGUMENT;
    argmax_kernel<<<dim3(rows), dim3(SAMPLE_THREADS), 0, stream>>>(logits, ld, vocab, out);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- temperature / top-k / top-p
struct SelectState {
    uint32_t prefix;                   // the bytes of the key chosen so far (high bytes)
    unsigned long long count_above;    // entries with a larger key than the prefix admits
    unsigned long long mass_above;     // their summed weights
};

// One radix select over the row.  by_mass == 0: the target-th largest entry (target >= 1).
// by_mass == 1: the first entry, in descending order, whose inclusive prefix sum of weights
// reaches target.  On return st.prefix is that entry's key and the two sums count what is
// strictly larger.
__device__ void radix_select(const float *row, int vocab, float max_logit, float inv_t, int by_mass,
                             unsigned long long target, SelectState &st, unsigned int *cnt,
                             unsigned long long *mass, SelectState *shared_st) {
    st.prefix = 0; st.count_above = 0; st.mass_above = 0;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        for (int d = threadIdx.x; d < 256; d += blockDim.x) { cnt[d] = 0; mass[d] = 0; }
        __syncthreads();
        for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
            const float v = row[i];
            const uint32_t k = order_key(v);
            if (pass > 0 && (k >> (shift + 8)) != (st.prefix >> (shift + 8))) continue;
            const int d = (k >> shift) & 255;
            atomicAdd(&cnt[d], 1u);
            atomicAdd(&mass[d], fixed_weight(v, max_logit, inv_t));
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            SelectState s = st;
            int chosen = -1, last_nonempty = -1;
            for (int d = 255; d >= 0; --d) {
                if (!cnt[d]) continue;
                last_nonempty = d;
                const unsigned long long have = by_mass ? s.mass_above + mass[d] : s.count_above + cnt[d];
                if (have >= target) { chosen = d; break; }
                s.count_above += cnt[d];
                s.mass_above += mass[d];
            }
            if (chosen < 0) {          // the target lies beyond the row's total: take the last entry
                chosen = last_nonempty < 0 ? 0 : last_nonempty;
                if (last_nonempty >= 0) { s.count_above -= cnt[chosen]; s.mass_above -= mass[chosen]; }
            }
            s.prefix = st.prefix | ((uint32_t)chosen << shift);
            *shared_st = s;
        }
        __syncthreads();
        st = *shared_st;
        __syncthreads();
    }
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float *__restrict__ logits, int ld, int vocab, const float *__restrict__ temperature,
              const float *__restrict__ top_p, const int *__restrict__ top_k, const float *__restrict__ uniform,
              int *__restrict__ out) {
    __shared__ unsigned int cnt[256];
    __shared__ unsigned long long mass[256];
    __shared__ SelectState shared_st;
    __shared__ float red[SAMPLE_THREADS / WAVE];
    __shared__ unsigned long long red64[SAMPLE_THREADS / WAVE];
    __shared__ int seg_count[SAMPLE_THREADS];
    __shared__ int result;

    const int r = blockIdx.x;
    const float *row = logits + (size_t)r * ld;
    const float inv_t = 1.0f / temperature[r];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int nwaves = blockDim.x / WAVE;

    // the largest logit
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) mx = fmaxf(mx, row[i]);
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = red[0];
    for (int w = 1; w < nwaves; ++w) mx = fmaxf(mx, red[w]);
    __syncthreads();

    // the sum of all weights
    unsigned long long total = 0;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) total += fixed_weight(row[i], mx, inv_t);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) total += __shfl_xor(total, off, WAVE);
    if (lane == 0) red64[wave] = total;
    __syncthreads();
    total = 0;
    for (int w = 0; w < nwaves; ++w) total += red64[w];
    __syncthreads();

    // c[top_k - 1]: the weights of the top_k largest entries
    SelectState st;
    unsigned long long limit_k = total;
    int k = top_k[r];
    if (k >= 1 && k < vocab) {
        radix_select(row, vocab, mx, inv_t, 0, (unsigned long long)k, st, cnt, mass, &shared_st);
        const unsigned long long w_tie = fixed_weight(key_value(st.prefix), mx, inv_t);
        limit_k = st.mass_above + ((unsigned long long)k - st.count_above) * w_tie;
    }
    // p = u * min(top_p * c[n-1], c[top_k-1])
    const double lim_p = (double)top_p[r] * (double)total;
    const double lim = lim_p < (double)limit_k ? lim_p : (double)limit_k;
    unsigned long long target = (unsigned long long)((double)uniform[r] * lim);
    if (target > total) target = total;

    radix_select(row, vocab, mx, inv_t, 1, target, st, cnt, mass, &shared_st);

    // among equal logits: the m-th in index order, m = ceil((p - mass_above) / w)
    const uint32_t key = st.prefix;
    const unsigned long long w_tie = fixed_weight(key_value(key), mx, inv_t);
    unsigned long long m = 1;
    if (w_tie > 0 && target > st.mass_above) m = (target - st.mass_above + w_tie - 1) / w_tie;
    if (m < 1) m = 1;
    const int seg = (vocab + blockDim.x - 1) / blockDim.x;
    const int lo = threadIdx.x * seg, hi = (lo + seg < vocab) ? lo + seg : vocab;
    int mine = 0;
    for (int i = lo; i < hi; ++i) mine += order_key(row[i]) == key;
    seg_count[threadIdx.x] = mine;
    if (threadIdx.x == 0) result = -1;
    __syncthreads();
    if (threadIdx.x == 0) {
        // exclusive prefix counts, serial: 1024 additions
        int run = 0;
        for (int t = 0; t < (int)blockDim.x; ++t) { const int c = seg_count[t]; seg_count[t] = run; run += c; }
        red64[0] = (unsigned long long)run;
    }
    __syncthreads();
    const unsigned long long n_ties = red64[0];
    if (m > n_ties) m = n_ties;
    const int before = seg_count[threadIdx.x];
    if (mine > 0 && (unsigned long long)before < m && m <= (unsigned long long)(before + mine)) {
        int seen = before;
        for (int i = lo; i < hi; ++i)
            if (order_key(row[i]) == key && (unsigned long long)(++seen) == m) { result = i; break; }
    }
    __syncthreads();
    if (threadIdx.x == 0) out[r] = result < 0 ? 0 : result;
}

// One draw per row: temperature[r] > 0, 0 < top_p[r] <= 1, top_k[r] >= 1 (>= vocab: no cut),
// uniform[r] in [0, 1).  All arrays are on the device.
LCU_API int lcu_sample(const float *logits, int ld, int rows, int vocab, const float *temperature, const float *top_p,
                       const int *top_k, const float *uniform, int *out, hipStream_t stream) {
    if (rows <= 0) return LCU_OK;
    if (vocab <= 0 || vocab > MAX_VOCAB || ld < vocab) return LCU_BAD_ARGUMENT;
    sample_kernel<<<dim3(rows), dim3(SAMPLE_THREADS), 0, stream>>>(logits, ld, vocab, temperature, top_p, top_k, uniform, out);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
