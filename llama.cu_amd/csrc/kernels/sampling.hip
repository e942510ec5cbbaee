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
    // ascending float order -> ascending unsigned order; -0 counts as +0 (equal values are ordered
    // by index, as a stable sort by value orders them)
    const uint32_t u = x == 0.0f ? 0u : __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ unsigned long long fixed_weight(float logit, float max_logit, float inv_t) {
    const float w = expf((logit - max_logit) * inv_t);
    return (unsigned long long)((double)w * FIXED_ONE);
}

// A row is cut into `parts` stretches, one workgroup each; their borders are multiples of four
// logits.
__device__ __forceinline__ void part_range(int vocab, int part, int parts, int &lo, int &hi) {
    const int quads = (vocab + 3) / 4;
    lo = (int)((long long)quads * part / parts) * 4;
    hi = (int)((long long)quads * (part + 1) / parts) * 4;
    hi = hi < vocab ? hi : vocab;
}

// Every element of the stretch [lo, hi) of a row (lo a multiple of 4), for the threads of a block
// together: four neighbouring logits per load where the row allows it and several loads in flight
// (a stretch is read by one workgroup, so latency, not bandwidth, is what counts).  f(index,
// value); no order is promised.
template <class F>
__device__ __forceinline__ void scan_part(const float *__restrict__ row, int lo, int hi, F f) {
    const int vec_end = (((size_t)row % 16) == 0) ? lo + ((hi - lo) / 4) * 4 : lo;
#pragma unroll 4
    for (int i = lo + threadIdx.x * 4; i < vec_end; i += blockDim.x * 4) {
        const float4 v = *(const float4 *)(row + i);
        f(i, v.x); f(i + 1, v.y); f(i + 2, v.z); f(i + 3, v.w);
    }
    for (int i = vec_end + threadIdx.x; i < hi; i += blockDim.x) f(i, row[i]);
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
    int lo, hi;
    part_range(vocab, part, parts, lo, hi);
    float best = -INFINITY;
    int bi = 0x7fffffff;
    scan_part(row, lo, hi, [&](int i, float v) {
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    });
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

// One digit of a radix select, on the histograms of that digit in `sc` (every thread of the block
// must call it).  by_mass == 0: towards the target-th largest entry (target >= 1).  by_mass == 1:
// towards the first entry, in descending order, whose inclusive prefix sum of weights reaches the
// target.  `st` holds the digits chosen so far and what lies strictly above them; it is updated.
// The target of the first digit of a select by mass may depend on the row's total weight, which
// only this histogram tells: target_of(total) is asked once all bins are added up.
template <class TargetOf>
__device__ void walk_bins(int pass, int by_mass, TargetOf target_of, SelectState &st, SelectScratch &sc) {
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, nwaves = blockDim.x / WAVE;
    const int shift = select_shift(pass), bits = select_bits(pass), nbins = 1 << bits;
    if (threadIdx.x == 0) { sc.best = SELECT_BINS; sc.last_nonempty = -1; }
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
    const unsigned long long target = target_of(m_all);
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

// ---- the draw, in several launches
// A long row is more work than one workgroup should do alone (every logit is added to two
// histograms per digit): a row is cut into `parts` stretches, one workgroup each.  The stretches'
// histograms are added up in memory, and between the digits a small kernel with one workgroup per
// row walks the bins.  What a row's launches hand to each other lies in RowState and in the
// histograms [rows][SELECT_BINS], all zero at the start; a walk clears the bins it has read.
struct RowState {
    unsigned int max_key;              // order_key of the row's largest logit
    int pad;                           // (keeps the 64-bit members aligned)
    unsigned long long total;          // the sum of all weights
    unsigned long long limit_k;        // c[top_k - 1]: the weights of the top_k largest entries
    unsigned long long target;         // the point of the cumulative weights that was drawn
    SelectState st;                    // the select that is under way, or its result
};

__device__ __forceinline__ bool row_cuts_at_k(int k, int vocab) { return k >= 1 && k < vocab; }

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_max_kernel(const float *__restrict__ logits, int ld, int vocab, RowState *__restrict__ state) {
    __shared__ float red[SAMPLE_THREADS / WAVE];
    const int r = blockIdx.x;
    int lo, hi;
    part_range(vocab, blockIdx.y, gridDim.y, lo, hi);
    float mx = -INFINITY;
    scan_part(logits + (size_t)r * ld, lo, hi, [&](int, float v) { mx = fmaxf(mx, v); });
    mx = wave_max(mx);
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x / WAVE); ++w) mx = fmaxf(mx, red[w]);
        atomicMax(&state[r].max_key, order_key(mx));
    }
}

// The histograms of one digit over a stretch of a row, added to the row's histograms in memory.
// which == 0: the select by count that finds the top_k-th entry (rows without such a cut do
// nothing); which == 1: the select by weight that finds the drawn entry.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_hist_kernel(const float *__restrict__ logits, int ld, int vocab, const float *__restrict__ temperature,
                   const int *__restrict__ top_k, const RowState *__restrict__ state, int pass, int which,
                   unsigned int *__restrict__ hist_cnt, unsigned long long *__restrict__ hist_mass) {
    __shared__ unsigned int cnt[SELECT_BINS];
    __shared__ unsigned long long mass[SELECT_BINS];
    const int r = blockIdx.x;
    if (which == 0 && !row_cuts_at_k(top_k[r], vocab)) return;
    const float mx = key_value(state[r].max_key), inv_t = 1.0f / temperature[r];
    const uint32_t fixed = state[r].st.prefix;
    const int shift = select_shift(pass), bits = select_bits(pass), nbins = 1 << bits, above = shift + bits;
    for (int d = threadIdx.x; d < nbins; d += blockDim.x) { cnt[d] = 0; mass[d] = 0; }
    __syncthreads();
    int lo, hi;
    part_range(vocab, blockIdx.y, gridDim.y, lo, hi);
    scan_part(logits + (size_t)r * ld, lo, hi, [&](int, float v) {
        const uint32_t k = order_key(v);
        if (pass > 0 && (k >> above) != (fixed >> above)) return;
        const int d = (k >> shift) & (nbins - 1);
        atomicAdd(&cnt[d], 1u);
        atomicAdd(&mass[d], fixed_weight(v, mx, inv_t));
    });
    __syncthreads();
    for (int d = threadIdx.x; d < nbins; d += blockDim.x)
        if (cnt[d]) {
            atomicAdd(&hist_cnt[(size_t)r * SELECT_BINS + d], cnt[d]);
            atomicAdd(&hist_mass[(size_t)r * SELECT_BINS + d], mass[d]);
        }
}

// Between two digits: one workgroup per row takes the row's histograms (and clears them), walks
// the bins and writes the select's new state.  After the last digit of the select by count it
// turns the result into limit_k; before the first digit of the select by weight it makes the
// target, p = u * min(top_p * c[n-1], c[top_k-1]), from the total that this histogram gives.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_walk_kernel(int vocab, const float *__restrict__ temperature, const float *__restrict__ top_p,
                   const int *__restrict__ top_k, const float *__restrict__ uniform, RowState *__restrict__ state, int pass,
                   int which, unsigned int *__restrict__ hist_cnt, unsigned long long *__restrict__ hist_mass) {
    __shared__ SelectScratch sc;
    const int r = blockIdx.x;
    const int k = top_k[r];
    const bool cuts = row_cuts_at_k(k, vocab);
    if (which == 0 && !cuts) return;
    const int nbins = 1 << select_bits(pass);
    for (int d = threadIdx.x; d < SELECT_BINS; d += blockDim.x) {
        const bool in = d < nbins;
        sc.cnt[d] = in ? hist_cnt[(size_t)r * SELECT_BINS + d] : 0u;
        sc.mass[d] = in ? hist_mass[(size_t)r * SELECT_BINS + d] : 0ull;
        if (in) { hist_cnt[(size_t)r * SELECT_BINS + d] = 0u; hist_mass[(size_t)r * SELECT_BINS + d] = 0ull; }
    }
    RowState &rs = state[r];
    SelectState st = rs.st;
    if (pass == 0) { st.prefix = 0; st.count_above = 0; st.mass_above = 0; }
    const float top_p_r = top_p[r], u_r = uniform[r];
    const unsigned long long limit_k = rs.limit_k, old_target = rs.target;
    __syncthreads();
    unsigned long long total = 0, target = 0;
    walk_bins(pass, which, [&](unsigned long long all) -> unsigned long long {
        if (which == 0) return (unsigned long long)k;
        if (pass > 0) return old_target;
        total = all;                                   // nothing lies above the first digit: all bins are the row
        const double lim_p = (double)top_p_r * (double)total;
        const double lim_k = cuts ? (double)limit_k : (double)total;
        const double lim = lim_p < lim_k ? lim_p : lim_k;
        target = (unsigned long long)((double)u_r * lim);
        if (target > total) target = total;
        return target;
    }, st, sc);
    if (threadIdx.x == 0) {
        rs.st = st;
        if (which == 1 && pass == 0) { rs.total = total; rs.target = target; }
        if (which == 0 && pass == SELECT_PASSES - 1) {
            const float mx = key_value(rs.max_key), inv_t = 1.0f / temperature[r];
            const unsigned long long w_tie = fixed_weight(key_value(st.prefix), mx, inv_t);
            rs.limit_k = st.mass_above + ((unsigned long long)k - st.count_above) * w_tie;
        }
    }
}

// How many logits of each stretch have the chosen key, and the first of them.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_count_kernel(const float *__restrict__ logits, int ld, int vocab, const RowState *__restrict__ state,
                    int *__restrict__ part_count, int *__restrict__ part_first) {
    __shared__ int n_found, first_found;
    const int r = blockIdx.x;
    const uint32_t key = state[r].st.prefix;
    if (threadIdx.x == 0) { n_found = 0; first_found = 0x7fffffff; }
    __syncthreads();
    int lo, hi;
    part_range(vocab, blockIdx.y, gridDim.y, lo, hi);
    int seen_here = 0, first_here = 0x7fffffff;
    scan_part(logits + (size_t)r * ld, lo, hi, [&](int i, float v) {
        if (order_key(v) == key) { ++seen_here; first_here = i < first_here ? i : first_here; }
    });
    if (seen_here) { atomicAdd(&n_found, seen_here); atomicMin(&first_found, first_here); }
    __syncthreads();
    if (threadIdx.x == 0) {
        part_count[r * gridDim.y + blockIdx.y] = n_found;
        part_first[r * gridDim.y + blockIdx.y] = first_found;
    }
}

// Among equal logits: the m-th in index order, m = ceil((p - mass_above) / w).  Mostly one logit
// has the key; else the stretch that holds the m-th is counted thread by thread.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_pick_kernel(const float *__restrict__ logits, int ld, int vocab, const float *__restrict__ temperature,
                   const RowState *__restrict__ state, const int *__restrict__ part_count,
                   const int *__restrict__ part_first, int parts, int *__restrict__ out) {
    __shared__ int seg_count[SAMPLE_THREADS];
    __shared__ int result;
    const int r = blockIdx.x;
    const float *row = logits + (size_t)r * ld;
    const RowState &rs = state[r];
    const uint32_t key = rs.st.prefix;
    const float mx = key_value(rs.max_key), inv_t = 1.0f / temperature[r];
    const unsigned long long w_tie = fixed_weight(key_value(key), mx, inv_t);
    unsigned long long m = 1;
    if (w_tie > 0 && rs.target > rs.st.mass_above) m = (rs.target - rs.st.mass_above + w_tie - 1) / w_tie;
    if (m < 1) m = 1;
    unsigned long long n_ties = 0;
    int first = 0x7fffffff;
    for (int p = 0; p < parts; ++p) {
        n_ties += (unsigned long long)part_count[r * parts + p];
        first = part_first[r * parts + p] < first ? part_first[r * parts + p] : first;
    }
    if (n_ties <= 1) {
        if (threadIdx.x == 0) out[r] = n_ties == 1 ? first : 0;
        return;
    }
    if (m > n_ties) m = n_ties;
    // the stretch that holds the m-th, and how many lie before it
    int part = 0;
    unsigned long long before_part = 0;
    while (part + 1 < parts && before_part + (unsigned long long)part_count[r * parts + part] < m) {
        before_part += (unsigned long long)part_count[r * parts + part];
        ++part;
    }
    int p_lo, p_hi;
    part_range(vocab, part, parts, p_lo, p_hi);
    if (threadIdx.x == 0) result = -1;
    const int seg = (p_hi - p_lo + (int)blockDim.x - 1) / (int)blockDim.x;
    const int lo = p_lo + threadIdx.x * seg, hi = (lo + seg < p_hi) ? lo + seg : p_hi;
    int mine = 0;
    for (int i = lo; i < hi; ++i) mine += order_key(row[i]) == key;
    seg_count[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        // exclusive prefix counts, serial: 1024 additions
        int run = 0;
        for (int t = 0; t < (int)blockDim.x; ++t) { const int c = seg_count[t]; seg_count[t] = run; run += c; }
    }
    __syncthreads();
    const unsigned long long before = before_part + (unsigned long long)seg_count[threadIdx.x];
    if (mine > 0 && before < m && m <= before + (unsigned long long)mine) {
        unsigned long long seen = before;
        for (int i = lo; i < hi; ++i)
            if (order_key(row[i]) == key && ++seen == m) { result = i; break; }
    }
    __syncthreads();
    if (threadIdx.x == 0) out[r] = result < 0 ? 0 : result;
}

// Bytes of scratch memory that lcu_sample needs for `rows` rows cut in `parts` (zeroed by the caller).
LCU_API size_t lcu_sample_scratch_bytes(int rows, int parts) {
    if (rows <= 0 || parts <= 0) return 0;
    return (size_t)rows * (sizeof(RowState) + SELECT_BINS * (sizeof(unsigned int) + sizeof(unsigned long long)) +
                           2 * (size_t)parts * sizeof(int)) + 256;
}

// One draw per row: temperature[r] > 0, 0 < top_p[r] <= 1, top_k[r] >= 1 (>= vocab: no cut),
// uniform[r] in [0, 1).  All arrays are on the device.  any_top_k: some row has top_k < vocab
// (else the launches of that select are left out).  parts: workgroups per row (1 to 64);
// scratch: lcu_sample_scratch_bytes(rows, parts) bytes, 16-byte aligned, all zero.
LCU_API int lcu_sample(const float *logits, int ld, int rows, int vocab, const float *temperature, const float *top_p,
                       const int *top_k, const float *uniform, int *out, int any_top_k, int parts, void *scratch,
                       hipStream_t stream) {
    if (rows <= 0) return LCU_OK;
    if (vocab <= 0 || vocab > MAX_VOCAB || ld < vocab || parts < 1 || parts > 64 || !scratch || ((size_t)scratch & 15))
        return LCU_BAD_ARGUMENT;
    char *at = (char *)scratch;
    unsigned long long *hist_mass = (unsigned long long *)at; at += (size_t)rows * SELECT_BINS * sizeof(unsigned long long);
    RowState *state = (RowState *)at;                         at += (size_t)rows * sizeof(RowState);
    unsigned int *hist_cnt = (unsigned int *)at;              at += (size_t)rows * SELECT_BINS * sizeof(unsigned int);
    int *part_count = (int *)at;                              at += (size_t)rows * parts * sizeof(int);
    int *part_first = (int *)at;
    const dim3 cut(rows, parts), whole(rows), block(SAMPLE_THREADS);
    sample_max_kernel<<<cut, block, 0, stream>>>(logits, ld, vocab, state);
    for (int which = any_top_k ? 0 : 1; which < 2; ++which)
        for (int pass = 0; pass < SELECT_PASSES; ++pass) {
            sample_hist_kernel<<<cut, block, 0, stream>>>(logits, ld, vocab, temperature, top_k, state, pass, which, hist_cnt,
                                                         hist_mass);
            sample_walk_kernel<<<whole, block, 0, stream>>>(vocab, temperature, top_p, top_k, uniform, state, pass, which,
                                                           hist_cnt, hist_mass);
        }
    sample_count_kernel<<<cut, block, 0, stream>>>(logits, ld, vocab, state, part_count, part_first);
    sample_pick_kernel<<<whole, block, 0, stream>>>(logits, ld, vocab, temperature, state, part_count, part_first, parts, out);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- the chosen token's log-probability
// out[r] = logits[r][tokens[r]] - log(sum_j exp(logits[r][j])), the natural logarithm of the token's probability under
// the softmax of the row at temperature 1 (what the model itself gives the token, whatever the draw's temperature and
// cuts were).  One workgroup a row; the maximum first, then the sum of exp(l - max) in a fixed order.  A token outside
// the row gives NaN.
__global__ void __launch_bounds__(SAMPLE_THREADS)
token_logprob_kernel(const float *__restrict__ logits, int ld, int vocab, const int *__restrict__ tokens, float *__restrict__ out) {
    __shared__ float scratch[16];
    const float *row = logits + (size_t)blockIdx.x * ld;
    float mx = -INFINITY;
    scan_part(row, 0, vocab, [&](int, float v) { mx = fmaxf(mx, v); });
    mx = wave_max(mx);
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    if (lane == 0) scratch[wave] = mx;
    __syncthreads();
    mx = scratch[0];
    for (int i = 1; i < SAMPLE_THREADS / WAVE; ++i) mx = fmaxf(mx, scratch[i]);
    float sum = 0.f;
    scan_part(row, 0, vocab, [&](int, float v) { sum += expf(v - mx); });
    sum = block_sum(sum, scratch);
    if (threadIdx.x == 0) {
        const int t = tokens[blockIdx.x];
        out[blockIdx.x] = (t >= 0 && t < vocab) ? row[t] - mx - logf(sum) : NAN;
    }
}

// logits: [rows, ld] float32 with vocab <= ld; tokens: [rows] int32; out: [rows] float32.
LCU_API int lcu_token_logprob(const float *logits, int ld, int rows, int vocab, const int *tokens, float *out, hipStream_t stream) {
    if (rows <= 0) return LCU_OK;
    if (vocab <= 0 || ld < vocab || !logits || !tokens || !out) return LCU_BAD_ARGUMENT;
    token_logprob_kernel<<<dim3(rows), dim3(SAMPLE_THREADS), 0, stream>>>(logits, ld, vocab, tokens, out);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
