// Sampling from rows of float32 logits: arg-max, and temperature sampling with
// top-k and top-p cuts.
//
// The reference sorts a row descending, sets w_0 = 1 and w_i = exp((l_i - l_0)/T),
// takes inclusive prefix sums c, draws p = u * min(top_p * c[n-1], c[top_k-1]) and
// returns the first entry with c[i] >= p (llama.cu/src/op/random_sample/sample.cuh:71-87,
// 186-207, with library sort, scan and reduce).  The same token comes out here without
// sorting: the entry with c[i] >= p is found by a radix select over the bit patterns of
// the logits, most significant digit first, on histograms of counts and of weights.
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

// Every element of a row, for the threads of a block together: four neighbouring logits per
// load where the row allows it and several loads in flight (a row is read by one workgroup,
// so latency, not bandwidth, is what counts).  f(index, value); no order is promised.
template <class F>
__device__ __forceinline__ void scan_row(const float *__restrict__ row, int vocab, F f) {
    const int vec_end = (((size_t)row % 16) == 0) ? (vocab / 4) * 4 : 0;
#pragma unroll 4
    for (int i = threadIdx.x * 4; i < vec_end; i += blockDim.x * 4) {
        const float4 v = *(const float4 *)(row + i);
        f(i, v.x); f(i + 1, v.y); f(i + 2, v.z); f(i + 3, v.w);
    }
    for (int i = vec_end + threadIdx.x; i < vocab; i += blockDim.x) f(i, row[i]);
}

// ---------------------------------------------------------------- arg-max
// The largest logit of each row; among equals the lowest index.  NaN never wins.  A row is cut
// into gridDim.y parts, one workgroup each (a single workgroup reads a long row at the speed of
// one compute unit); with more than one part the parts' winners go to part_val / part_idx
// [rows][parts] and argmax_merge_kernel picks among them.
__global__ void __launch_bounds__(SAMPLE_THREADS)
argmax_kernel(const float *__restrict__ logits, int ld, int vocab, int *__restrict__ out, float *__restrict__ part_val,
              int *__restrict__ part_idx) {
    const float *row = logits + (size_t)blockIdx.x * ld;
    const int parts = gridDim.y, part = blockIdx.y;
    // the part's share of the row, in units of four logits
    const int quads = (vocab + 3) / 4;
    const int lo = (int)((long long)quads * part / parts) * 4;
    int hi = (int)((long long)quads * (part + 1) / parts) * 4;
    hi = hi < vocab ? hi : vocab;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    // four neighbouring logits per load where the row allows it (many loads in flight: latency,
    // not bandwidth, is what counts)
    const int vec_end = (((size_t)row % 16) == 0) ? lo + ((hi - lo) / 4) * 4 : lo;
#pragma unroll 4
    for (int i = lo + threadIdx.x * 4; i < vec_end; i += blockDim.x * 4) {
        const float4 v = *(const float4 *)(row + i);
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (e[k] > best || (e[k] == best && i + k < bi)) { best = e[k]; bi = i + k; }
    }
    for (int i = vec_end + threadIdx.x; i < hi; i += blockDim.x) {
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
        if (parts == 1) {
            out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
        } else {
            part_val[(size_t)blockIdx.x * parts + part] = best;
            part_idx[(size_t)blockIdx.x * parts + part] = bi;
        }
    }
}

__global__ void argmax_merge_kernel(const float *__restrict__ part_val, const int *__restrict__ part_idx, int parts,
                                    int *__restrict__ out) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int p = threadIdx.x; p < parts; p += WAVE) {
        const float v = part_val[(size_t)blockIdx.x * parts + p];
        const int i = part_idx[(size_t)blockIdx.x * parts + p];
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, WAVE);
        const int oi = __shfl_xor(bi, off, WAVE);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// parts: into how many workgroups a row is cut (1: one kernel, no scratch); part_val, part_idx:
// [rows * parts] when parts > 1.
LCU_API int lcu_argmax(const float *logits, int ld, int rows, int vocab, int *out, int parts, float *part_val, int *part_idx,
                       hipStream_t stream) {
    if (rows <= 0) return LCU_OK;
    if (vocab <= 0 || ld < vocab || parts < 1 || parts > 1024 || (parts > 1 && (!part_val || !part_idx))) return LCU_BAD_ARGUMENT;
    argmax_kernel<<<dim3(rows, parts), dim3(SAMPLE_THREADS), 0, stream>>>(logits, ld, vocab, out, part_val, part_idx);
    LCU_LAUNCH_CHECK();
    if (parts > 1) {
        argmax_merge_kernel<<<dim3(rows), dim3(WAVE), 0, stream>>>(part_val, part_idx, parts, out);
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}

// ---------------------------------------------------------------- temperature / top-k / top-p
struct SelectState {
    uint32_t prefix;                   // the bytes of the key chosen so far (high bytes)
    unsigned long long count_above;    // entries with a larger key than the prefix admits
    unsigned long long mass_above;     // their summed weights
};

// The digits of the radix select, most significant first: 12, 12 and 8 bits.  The first digit
// holds the sign, the exponent and three bits of the mantissa: with one byte (sign and seven
// bits of the exponent) nearly all logits of a row fall into a handful of bins and their
// atomic additions queue up behind each other.
constexpr int SELECT_PASSES = 3;
constexpr int SELECT_BINS = 4096;
__device__ __forceinline__ int select_shift(int pass) { return pass == 0 ? 20 : (pass == 1 ? 8 : 0); }
__device__ __forceinline__ int select_bits(int pass) { return pass == 2 ? 8 : 12; }

struct SelectScratch {
    unsigned int cnt[SELECT_BINS];
    unsigned long long mass[SELECT_BINS];
    unsigned int wave_cnt[SAMPLE_THREADS / WAVE];
    unsigned long long wave_mass[SAMPLE_THREADS / WAVE];
    int best, last_nonempty;
    SelectState st;
};

// One radix select over the row.  by_mass == 0: the target-th largest entry (target >= 1).
// by_mass == 1: the first entry, in descending order, whose inclusive prefix sum of weights
// reaches target.  On return st.prefix is that entry's key and the two sums count what is
// strictly larger.  Every thread of the block must call it.
__device__ void radix_select(const float *row, int vocab, float max_logit, float inv_t, int by_mass,
                             unsigned long long target, SelectState &st, SelectScratch &sc) {
    st.prefix = 0; st.count_above = 0; st.mass_above = 0;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, nwaves = blockDim.x / WAVE;
    for (int pass = 0; pass < SELECT_PASSES; ++pass) {
        const int shift = select_shift(pass), bits = select_bits(pass), nbins = 1 << bits;
        for (int d = threadIdx.x; d < SELECT_BINS; d += blockDim.x) { sc.cnt[d] = 0; sc.mass[d] = 0; }
        if (threadIdx.x == 0) { sc.best = SELECT_BINS; sc.last_nonempty = -1; }
        __syncthreads();
        const int above = shift + bits;                      // the bits that earlier passes have fixed
        const uint32_t fixed = st.prefix;
        scan_row(row, vocab, [&](int, float v) {
            const uint32_t k = order_key(v);
            if (pass > 0 && (k >> above) != (fixed >> above)) return;
            const int d = (k >> shift) & (nbins - 1);
            atomicAdd(&sc.cnt[d], 1u);
            atomicAdd(&sc.mass[d], fixed_weight(v, max_logit, inv_t));
        });
        __syncthreads();
        // Walk the bins from the largest digit down, all threads together: thread t has the
        // places 4t .. 4t+3 of that walk (place q is digit nbins-1-q); an exclusive scan over
        // the threads gives what lies above its places.
        const int per = SELECT_BINS / SAMPLE_THREADS;
        unsigned int c_mine = 0;
        unsigned long long m_mine = 0;
#pragma unroll
        for (int e = 0; e < per; ++e) {
            const int q = threadIdx.x * per + e;
            if (q < nbins) { c_mine += sc.cnt[nbins - 1 - q]; m_mine += sc.mass[nbins - 1 - q]; }
        }
        unsigned int c_scan = c_mine;
        unsigned long long m_scan = m_mine;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const unsigned int c_up = __shfl_up(c_scan, off, WAVE);
            const unsigned long long m_up = __shfl_up(m_scan, off, WAVE);
            if (lane >= off) { c_scan += c_up; m_scan += m_up; }
        }
        if (lane == WAVE - 1) { sc.wave_cnt[wave] = c_scan; sc.wave_mass[wave] = m_scan; }
        __syncthreads();
        unsigned long long c_before = st.count_above, m_before = st.mass_above, c_all = 0, m_all = 0;
        for (int w = 0; w < nwaves; ++w) {
            if (w < wave) { c_before += sc.wave_cnt[w]; m_before += sc.wave_mass[w]; }
            c_all += sc.wave_cnt[w]; m_all += sc.wave_mass[w];
        }
        c_before += c_scan - c_mine;                         // exclusive within the wave
        m_before += m_scan - m_mine;
        bool found = false;
        unsigned long long c_at = 0, m_at = 0;
        int q_at = 0;
#pragma unroll
        for (int e = 0; e < per; ++e) {
            const int q = threadIdx.x * per + e;
            if (q >= nbins) break;
            const unsigned int c = sc.cnt[nbins - 1 - q];
            const unsigned long long m = sc.mass[nbins - 1 - q];
            if (c) {
                atomicMax(&sc.last_nonempty, q);
                const unsigned long long have = by_mass ? m_before + m : c_before + c;
                if (!found && have >= target) { found = true; c_at = c_before; m_at = m_before; q_at = q; }
            }
            c_before += c;
            m_before += m;
        }
        if (found) atomicMin(&sc.best, q_at);
        __syncthreads();
        if (sc.best < SELECT_BINS) {
            if (found && q_at == sc.best) {                   // exactly one thread: the owner of that place
                sc.st.prefix = st.prefix | ((uint32_t)(nbins - 1 - q_at) << shift);
                sc.st.count_above = c_at;
                sc.st.mass_above = m_at;
            }
        } else if (threadIdx.x == 0) {
            // the target lies beyond the row's total: take the last entry
            const int q = sc.last_nonempty < 0 ? nbins - 1 : sc.last_nonempty;
            const int d = nbins - 1 - q;
            sc.st.prefix = st.prefix | ((uint32_t)d << shift);
            sc.st.count_above = st.count_above + c_all - (sc.last_nonempty < 0 ? 0 : sc.cnt[d]);
            sc.st.mass_above = st.mass_above + m_all - (sc.last_nonempty < 0 ? 0 : sc.mass[d]);
        }
        __syncthreads();
        st = sc.st;
        __syncthreads();
    }
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float *__restrict__ logits, int ld, int vocab, const float *__restrict__ temperature,
              const float *__restrict__ top_p, const int *__restrict__ top_k, const float *__restrict__ uniform,
              int *__restrict__ out) {
    __shared__ SelectScratch sc;
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
    scan_row(row, vocab, [&](int, float v) { mx = fmaxf(mx, v); });
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = red[0];
    for (int w = 1; w < nwaves; ++w) mx = fmaxf(mx, red[w]);
    __syncthreads();

    // the sum of all weights
    unsigned long long total = 0;
    scan_row(row, vocab, [&](int, float v) { total += fixed_weight(v, mx, inv_t); });
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
        radix_select(row, vocab, mx, inv_t, 0, (unsigned long long)k, st, sc);
        const unsigned long long w_tie = fixed_weight(key_value(st.prefix), mx, inv_t);
        limit_k = st.mass_above + ((unsigned long long)k - st.count_above) * w_tie;
    }
    // p = u * min(top_p * c[n-1], c[top_k-1])
    const double lim_p = (double)top_p[r] * (double)total;
    const double lim = lim_p < (double)limit_k ? lim_p : (double)limit_k;
    unsigned long long target = (unsigned long long)((double)uniform[r] * lim);
    if (target > total) target = total;

    radix_select(row, vocab, mx, inv_t, 1, target, st, sc);

    // among equal logits: the m-th in index order, m = ceil((p - mass_above) / w)
    const uint32_t key = st.prefix;
    const unsigned long long w_tie = fixed_weight(key_value(key), mx, inv_t);
    unsigned long long m = 1;
    if (w_tie > 0 && target > st.mass_above) m = (target - st.mass_above + w_tie - 1) / w_tie;
    if (m < 1) m = 1;
    // Mostly one logit has that key: count them in a fast pass and take the one.
    __shared__ int n_found, first_found;
    if (threadIdx.x == 0) { n_found = 0; first_found = 0x7fffffff; result = -1; }
    __syncthreads();
    int seen_here = 0, first_here = 0x7fffffff;
    scan_row(row, vocab, [&](int i, float v) {
        if (order_key(v) == key) { ++seen_here; first_here = i < first_here ? i : first_here; }
    });
    if (seen_here) { atomicAdd(&n_found, seen_here); atomicMin(&first_found, first_here); }
    __syncthreads();
    if (n_found <= 1) {
        if (threadIdx.x == 0) result = n_found == 1 ? first_found : -1;
    } else {
        // several equal logits: the m-th in index order; every thread counts a stretch of the row
        const int seg = (vocab + blockDim.x - 1) / blockDim.x;
        const int lo = threadIdx.x * seg, hi = (lo + seg < vocab) ? lo + seg : vocab;
        int mine = 0;
        for (int i = lo; i < hi; ++i) mine += order_key(row[i]) == key;
        seg_count[threadIdx.x] = mine;
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
