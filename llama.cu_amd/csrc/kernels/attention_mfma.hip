// Causal attention over the paged cache on the matrix cores, for bfloat16.
//
// Both kernels work on the transposed problem, so that nothing has to move between
// lanes or through LDS between the two matrix products:
//   S^T[key, q] = K[key, :] . Q[q, :]      A = K (a lane holds 8 dims of one key: one 16-byte
//                                          load in the cache's key layout), B = Q (kept in registers)
//   O^T[dim, q] += V^T[dim, key] . P^T[key, q]   A = V^T (a lane holds tokens of one dim, as the
//                                          cache's value layout has them), B = P^T: exactly the
//                                          lane's own S^T values
// so the softmax's maximum and sum run over a lane's registers and one or two cross-lane steps.
// Which keys a lane holds is the kernel's choice, by the order in which it feeds the keys' rows
// to the first product.  Scores, the running maximum and sum and the output are 32-bit; P is
// rounded to bfloat16 for the second product.
//
// A "row" is one (token, head) pair; the rows of a block share a request and a key/value head:
// the heads of a group for one token, for several tokens if the group is small.
//
//   decode kernel   one token per request, v_mfma_f32_16x16x32_bf16 (blocks of 16 rows; a lane
//                   owns row lane % 16 and 8 of each 32 keys, 4 of each tile of 16, which are
//                   neighbours in memory).  A workgroup of 4 waves takes one request and
//                   key/value head and one of `n_splits` equal parts of its keys; the
//                   waves take 32-key steps in turn and merge through LDS; parts are
//                   merged by a second kernel.
//   prefill kernel  any number of tokens per request (also one), v_mfma_f32_32x32x16_bf16 (blocks
//                   of 32 rows; a lane owns row lane % 32 and 16 of each 32 keys).  A workgroup of
//                   4 waves takes consecutive tokens of one request; the keys and values of a
//                   step are copied to LDS once and shared by the waves.
#include <mutex>

#include <utility>

#include "attention_static.h"
#include "common.h"
#include "kv_layout.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) { return pack2_bf16(lo, hi); }
// 2^x by the hardware's instruction (inputs here are <= 0; 2^-inf = 0)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// What a wave carries through its keys, for QB blocks of 16 rows.
template <int DH, int QB>
struct AttnState {
    f32x4 o[QB][DH / 16];   // O^T: lane = (row lane%16, dims 16*dt + 4*(lane/16) + r)
    float m[QB];            // running maximum (in units of log2), the same in the 4 lane groups
    float l[QB];            // running sum over the lane's own keys only
};

template <int DH, int QB>
__device__ __forceinline__ void attn_init(AttnState<DH, QB> &st) {
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        st.m[b] = -INFINITY;
        st.l[b] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) st.o[b][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
}

// The lane's share of the keys and values of one step: the 32 keys k0 .. k0+31 (k0 a
// multiple of 32) of key/value head kvh, as two tiles of 16 keys.
template <int DH>
struct KVFrag {
    u32x4 k[2][DH / 32];    // tile t, dims 32*kb + 8*grp .. + 7 of key 16*t + lane%16
    u32x2 v[DH / 16][2];    // dim 16*dt + lane%16, keys 16*t + 4*grp .. + 3
};

// The decode kernel reads a request's keys and values once a step: its loads are non-temporal (see gemm_skinny.hip's
// stream_load), so that they do not displace the weights' neighbours and the rows in the caches.
constexpr int DEC_STREAM = 2;

// The numbers of the two pages that hold the keys k0 .. k0+15 and k0+16 .. k0+31 (k0 the same in
// all lanes: the table is read through the scalar unit).
__device__ __forceinline__ void kv_pages(int (&pid)[2], const int *__restrict__ bt, int max_pages, int page, int k0) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        int pi = (k0 + 16 * t) / page;
        pi = pi < max_pages ? pi : max_pages - 1;       // a tile beyond the context is masked; keep the read in bounds
        pid[t] = bt[pi];
    }
}

// The loads are buffer loads whose buffer is the page: page, head, token and slice of dims
// make a scalar offset, and the lane adds one offset for the keys and one for the values that
// are the same in every step, so no addresses are held in vector registers.  pid: kv_pages of
// k0, read a step earlier so that no load waits for the table.  A page holds less than 2 GiB
// (the host checks).
template <int DH>
__device__ __forceinline__ void load_kv(KVFrag<DH> &f, const bf16_t *__restrict__ cache, const int (&pid)[2], int page,
                                        size_t page_elems, int nkvh, int kvh, int k0, int l16, int grp) {
    constexpr uint32_t E = sizeof(bf16_t);
    const uint32_t k_lane = ((uint32_t)grp * page + l16) * 8 * E;       // keys: [dim/8][token][8]
    const uint32_t v_lane = ((uint32_t)l16 * page + 4 * grp) * E;       // values: [dim][token]
    const uint32_t k_head = (uint32_t)kvh * (DH / 8) * page * 8 * E;
    const uint32_t v_head = (uint32_t)(nkvh + kvh) * DH * page * E;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const __amdgpu_buffer_rsrc_t pg = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<bf16_t *>(cache + (size_t)pid[t] * page_elems), 0, (uint32_t)(page_elems * E), 0x00020000);
        // the token's place in the page goes into the lane's offset (one addition for the keys, one for
        // the values), so that the scalar offsets are the same in every step
        const uint32_t tok0 = (k0 + 16 * t) % page;
        const uint32_t k_off = k_lane + tok0 * 8 * E, v_off = v_lane + tok0 * E;
#pragma unroll
        for (int kb = 0; kb < DH / 32; ++kb)
            f.k[t][kb] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(pg, k_off, k_head + (uint32_t)(4 * kb) * page * 8 * E, DEC_STREAM));
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt)
            f.v[dt][t] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(pg, v_off, v_head + (uint32_t)(16 * dt) * page * E, DEC_STREAM));
    }
}

// The same loads with a full address in every lane (the block table is read by the lanes too).
template <int DH>
__device__ __forceinline__ void load_kv_flat(KVFrag<DH> &f, const bf16_t *__restrict__ cache, const int *__restrict__ bt,
                                             int max_pages, int page, size_t page_elems, int nkvh, int kvh, int k0, int l16,
                                             int grp) {
    const size_t v_off = (size_t)nkvh * DH * page + (size_t)kvh * DH * page + 4 * grp;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int j = k0 + 16 * t;
        int pi = j / page;
        pi = pi < max_pages ? pi : max_pages - 1;       // a tile beyond the context is masked; keep the read in bounds
        const bf16_t *pg = cache + (size_t)bt[pi] * page_elems;
        const int tok0 = j % page;
        const bf16_t *kp = pg + ((size_t)kvh * (DH / 8) * page + tok0 + l16) * 8;
#pragma unroll
        for (int kb = 0; kb < DH / 32; ++kb) f.k[t][kb] = __builtin_nontemporal_load((const u32x4 *)(kp + (size_t)(4 * kb + grp) * page * 8));
        const bf16_t *vp = pg + v_off + tok0;
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) f.v[dt][t] = __builtin_nontemporal_load((const u32x2 *)(vp + (size_t)(16 * dt + l16) * page));
    }
}

// One step of the online softmax on loaded keys and values, in three parts.  p_row / lo_row:
// the last and first key each of the lane's rows may see.  MASK: some row of the wave does
// not see all 32 keys; p_max / lo_min bound what any row sees (values of keys outside are not
// used at all, whatever the memory holds).
//
// S^T = K Q^T.  The four sums (two key tiles, QB blocks of rows) are independent chains of
// DH/32 dependent matrix instructions; they are issued in turn, so that an instruction's
// result (ready after about three instructions' time) is there when its chain goes on.
template <int DH, int QB>
__device__ __forceinline__ void attn_scores(const u32x4 (&k)[2][DH / 32], const u32x4 (&q)[QB][DH / 32], f32x4 (&s)[QB][2]) {
#pragma unroll
    for (int b = 0; b < QB; ++b) s[b][0] = s[b][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < DH / 32; ++kb)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int b = 0; b < QB; ++b) s[b][t] = mfma16(k[t][kb], q[b][kb], s[b][t]);
}

constexpr float RESCALE_SLACK = 6.0f;

// The largest of the values that the lanes l, l + 16, l + 32 and l + 48 hold, in all four of them.
// The rows of 16 lanes are swapped in the vector unit (v_permlane16_swap, v_permlane32_swap): a
// shuffle through LDS takes an order of magnitude longer, and the softmax waits for this value.
__device__ __forceinline__ float max_over_groups(float x) {
    const unsigned u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);     // (rows 0 0 2 2, rows 1 1 3 3)
    const unsigned v = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);     // (lower half twice, upper half twice)
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// The softmax of the step, online: new maxima and sums, the output rescaled, the weights as
// bfloat16 operands.
// The lane's eight scores are four keys of each tile, k0 + 16 t + 4 grp .. + 3.
template <int DH, int QB, bool MASK>
__device__ __forceinline__ void attn_softmax(const f32x4 (&s)[QB][2], int k0, AttnState<DH, QB> &st, const int (&p_row)[QB],
                                             const int (&lo_row)[QB], float scale_log2, int grp, u32x4 (&pb)[QB]) {
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        float v[8];
#pragma unroll
        for (int r = 0; r < 4; ++r) { v[r] = s[b][0][r]; v[4 + r] = s[b][1][r]; }
        if (MASK) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int j = k0 + 16 * (r / 4) + 4 * grp + (r % 4);
                if (j > p_row[b] || j < lo_row[b]) v[r] = -INFINITY;
            }
        }
        float mx = v[0];
#pragma unroll
        for (int r = 1; r < 8; ++r) mx = fmaxf(mx, v[r]);
        mx = max_over_groups(mx);
        // The reference point of the exponentials need not be the exact maximum: it moves only
        // when the maximum has grown by more than 2^RESCALE_SLACK, so the weights stay below
        // that and the output is rarely rescaled (the result is the same up to rounding).
        const float m_true = fmaxf(st.m[b], mx * scale_log2);
        const float m_new = m_true - st.m[b] <= RESCALE_SLACK ? st.m[b] : m_true;   // false for the first keys (-inf)
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = fast_exp2(st.m[b] - m_safe);
        float p[8], sum = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            p[r] = fast_exp2(fmaf(v[r], scale_log2, -m_safe));
            sum += p[r];
        }
        st.l[b] = st.l[b] * alpha + sum;
        st.m[b] = m_new;
        // the output is rescaled only when some row's maximum has moved (the same test in all lanes)
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int dt = 0; dt < DH / 16; ++dt) st.o[b][dt] *= alpha;
        }
        pb[b] = u32x4{pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
    }
}

// O^T += V^T P^T
template <int DH, int QB, bool MASK>
__device__ __forceinline__ void attn_mix(const u32x2 (&v)[DH / 16][2], const u32x4 (&pb)[QB], int k0, int p_max, int lo_min,
                                         int grp, AttnState<DH, QB> &st) {
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt) {
        u32x2 v0 = v[dt][0], v1 = v[dt][1];
        if (MASK) {
            // values of keys that no row sees are taken as zero: their memory may hold anything
            const int j0 = k0 + 4 * grp, j1 = k0 + 16 + 4 * grp;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t keep = (r & 1) ? 0x0000ffffu : 0xffff0000u;   // clears element r of its dword
                if (j0 + r > p_max || j0 + r < lo_min) { if (r < 2) v0.x &= keep; else v0.y &= keep; }
                if (j1 + r > p_max || j1 + r < lo_min) { if (r < 2) v1.x &= keep; else v1.y &= keep; }
            }
        }
        const u32x4 a = u32x4{v0.x, v0.y, v1.x, v1.y};
#pragma unroll
        for (int b = 0; b < QB; ++b) st.o[b][dt] = mfma16(a, pb[b], st.o[b][dt]);
    }
}

template <int DH, int QB, bool MASK>
__device__ __forceinline__ void attn_compute(const KVFrag<DH> &f, int k0, const u32x4 (&q)[QB][DH / 32],
                                             AttnState<DH, QB> &st, const int (&p_row)[QB], const int (&lo_row)[QB],
                                             int p_max, int lo_min, float scale_log2, int grp) {
    f32x4 s[QB][2];
    attn_scores<DH, QB>(f.k, q, s);
    u32x4 pb[QB];
    attn_softmax<DH, QB, MASK>(s, k0, st, p_row, lo_row, scale_log2, grp, pb);
    attn_mix<DH, QB, MASK>(f.v, pb, k0, p_max, lo_min, grp, st);
}

// Masks only where a row needs them (the choice is the same for the whole wave).
template <int DH, int QB>
__device__ __forceinline__ void attn_block(const KVFrag<DH> &f, int k0, bool mask, const u32x4 (&q)[QB][DH / 32],
                                           AttnState<DH, QB> &st, const int (&p_row)[QB], const int (&lo_row)[QB],
                                           int p_max, int lo_min, float scale_log2, int grp) {
    if (mask) attn_compute<DH, QB, true>(f, k0, q, st, p_row, lo_row, p_max, lo_min, scale_log2, grp);
    else attn_compute<DH, QB, false>(f, k0, q, st, p_row, lo_row, p_max, lo_min, scale_log2, grp);
}

// The lane's part of the queries of one block of rows: 8 dims of row lane%16 per 32-dim
// slice, zero for a row that does not exist.
template <int DH>
__device__ __forceinline__ void load_q(const bf16_t *__restrict__ qrow, bool valid, u32x4 (&q)[DH / 32], int grp) {
#pragma unroll
    for (int kb = 0; kb < DH / 32; ++kb)
        q[kb] = valid ? *(const u32x4 *)(qrow + 32 * kb + 8 * grp) : u32x4{0u, 0u, 0u, 0u};
}

// ============================================================================ decode
#ifndef LCU_DEC_WAVES
#define LCU_DEC_WAVES 4
#endif
constexpr int DEC_WAVES = LCU_DEC_WAVES;
#ifndef LCU_DEC_MIN_WAVES
#define LCU_DEC_MIN_WAVES 2      // two waves per SIMD: measured faster than one with more registers
#endif

template <int DH, bool FLAT>
__global__ void __launch_bounds__(DEC_WAVES *WAVE, LCU_DEC_MIN_WAVES)
attention_decode_kernel(const bf16_t *__restrict__ q, int q_stride, bf16_t *__restrict__ out, int out_stride,
                        const bf16_t *__restrict__ cache, const int *__restrict__ block_table, int max_pages,
                        const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                        const int *__restrict__ req_list, int nh, int nkvh, int page, float scale_log2, int window,
                        int n_splits, float *__restrict__ part_o, float *__restrict__ part_ml) {
    extern __shared__ float lds[];                 // [waves][16][DH] outputs, then [waves][16][2] (m, l)
    const int g = nh / nkvh;
    const int chunks = (g + 15) / 16;
    const int ri = blockIdx.x / (nkvh * chunks);
    const int r = req_list ? req_list[ri] : ri;         // the batch's decoding requests, or all of them
    const int kvh = (blockIdx.x / chunks) % nkvh;
    const int chunk = blockIdx.x % chunks;
    const int split = blockIdx.y;
    // the wave's number as a scalar: its steps' pages are then read through the scalar unit, and
    // no wait for a page number stands between the loads of keys and values in flight
    const int lane = threadIdx.x & (WAVE - 1), wave = FLAT ? threadIdx.x / WAVE : __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int l16 = lane & 15, grp = lane >> 4;
    const int rows = (g - 16 * chunk) < 16 ? (g - 16 * chunk) : 16;
    const int token = q_start[r];
    const int p = ctx_len[r] - 1;
    const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
    const int head0 = kvh * g + 16 * chunk;

    u32x4 qv[1][DH / 32];
    load_q<DH>(q + (size_t)token * q_stride + (size_t)(head0 + l16) * DH, l16 < rows, qv[0], grp);
    AttnState<DH, 1> st;
    attn_init(st);
    const int p_row[1] = {p}, lo_row[1] = {lo};
    const int *bt = block_table + (size_t)r * max_pages;
    const size_t page_elems = kv_page_elems(nkvh, DH, page);

    // this split's share of the 32-key steps, the waves in turn
    const int first = lo / 32, last = p / 32, nblk = last - first + 1;
    const int b0 = first + (int)((long long)nblk * split / n_splits);
    const int b1 = first + (int)((long long)nblk * (split + 1) / n_splits);
    // the wave's steps are blk, blk + 4, ...; the next step's loads are in flight while one is computed
    KVFrag<DH> fa, fb;
    if (FLAT) {
        int blk = b0 + wave;
        if (blk < b1) load_kv_flat<DH>(fa, cache, bt, max_pages, page, page_elems, nkvh, kvh, blk * 32, l16, grp);
        for (; blk < b1; blk += 2 * DEC_WAVES) {
            const int nb = blk + DEC_WAVES, nb2 = blk + 2 * DEC_WAVES;
            if (nb < b1) load_kv_flat<DH>(fb, cache, bt, max_pages, page, page_elems, nkvh, kvh, nb * 32, l16, grp);
            attn_block<DH, 1>(fa, blk * 32, blk * 32 + 31 > p || blk * 32 < lo, qv, st, p_row, lo_row, p, lo, scale_log2, grp);
            if (nb2 < b1) load_kv_flat<DH>(fa, cache, bt, max_pages, page, page_elems, nkvh, kvh, nb2 * 32, l16, grp);
            if (nb < b1)
                attn_block<DH, 1>(fb, nb * 32, nb * 32 + 31 > p || nb * 32 < lo, qv, st, p_row, lo_row, p, lo, scale_log2, grp);
        }
    } else {
        // the pages of the step after the next are already known
        int ida[2], idb[2];
        int blk = b0 + wave;
        kv_pages(ida, bt, max_pages, page, blk * 32);
        kv_pages(idb, bt, max_pages, page, (blk + DEC_WAVES) * 32);
        if (blk < b1) load_kv<DH>(fa, cache, ida, page, page_elems, nkvh, kvh, blk * 32, l16, grp);
        kv_pages(ida, bt, max_pages, page, (blk + 2 * DEC_WAVES) * 32);
        for (; blk < b1; blk += 2 * DEC_WAVES) {
            const int nb = blk + DEC_WAVES, nb2 = blk + 2 * DEC_WAVES;
            if (nb < b1) load_kv<DH>(fb, cache, idb, page, page_elems, nkvh, kvh, nb * 32, l16, grp);
            kv_pages(idb, bt, max_pages, page, (nb + 2 * DEC_WAVES) * 32);
            __builtin_amdgcn_sched_barrier(0);         // asked for before the arithmetic, there after it
            attn_block<DH, 1>(fa, blk * 32, blk * 32 + 31 > p || blk * 32 < lo, qv, st, p_row, lo_row, p, lo, scale_log2, grp);
            if (nb2 < b1) load_kv<DH>(fa, cache, ida, page, page_elems, nkvh, kvh, nb2 * 32, l16, grp);
            kv_pages(ida, bt, max_pages, page, (nb2 + 2 * DEC_WAVES) * 32);
            __builtin_amdgcn_sched_barrier(0);
            if (nb < b1)
                attn_block<DH, 1>(fb, nb * 32, nb * 32 + 31 > p || nb * 32 < lo, qv, st, p_row, lo_row, p, lo, scale_log2, grp);
        }
    }
    // ---- merge the waves
    float l_all = st.l[0];
    l_all += __shfl_xor(l_all, 16, WAVE);
    l_all += __shfl_xor(l_all, 32, WAVE);
    float *lds_o = lds;
    float *lds_ml = lds + DEC_WAVES * 16 * DH;
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) lds_o[((size_t)wave * 16 + l16) * DH + 16 * dt + 4 * grp + rr] = st.o[0][dt][rr];
    if (grp == 0) {
        lds_ml[(wave * 16 + l16) * 2 + 0] = st.m[0];
        lds_ml[(wave * 16 + l16) * 2 + 1] = l_all;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < rows * DH; idx += DEC_WAVES * WAVE) {
        const int row = idx / DH, d = idx % DH;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) M = fmaxf(M, lds_ml[(w * 16 + row) * 2]);
        const float M_safe = M == -INFINITY ? 0.f : M;
        float L = 0.f, val = 0.f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            const float f = exp2f(lds_ml[(w * 16 + row) * 2] - M_safe);
            L += lds_ml[(w * 16 + row) * 2 + 1] * f;
            val += lds_o[((size_t)w * 16 + row) * DH + d] * f;
        }
        const int head = head0 + row;
        if (n_splits == 1) {
            out[(size_t)token * out_stride + (size_t)head * DH + d] = from_f32<bf16_t>(val / L);
        } else {
            const size_t slot = ((size_t)ri * nh + head) * n_splits + split;
            part_o[slot * DH + d] = val;
            if (d == 0) { part_ml[slot * 2] = M; part_ml[slot * 2 + 1] = L; }
        }
    }
}

// Merges the parts of every (token, head): out = sum_s O_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// (A merge inside the decode kernel by the workgroup that finishes last needs a
// device-wide fence per workgroup, which writes back and invalidates the whole L2: measured
// several times slower than this second launch.)
template <int DH>
__global__ void __launch_bounds__(DH / 4)
attention_merge_kernel(bf16_t *__restrict__ out, int out_stride, const float *__restrict__ part_o,
                       const float *__restrict__ part_ml, const int *__restrict__ q_start,
                       const int *__restrict__ req_list, int nh, int n_splits) {
    // a thread has four dims of one (token, head); the loads of up to eight parts are issued
    // together, so the kernel takes one trip to memory and not one per part
    constexpr int GROUP = 8;
    const int ri = blockIdx.x, head = blockIdx.y, d0 = 4 * threadIdx.x;
    const int token = q_start[req_list ? req_list[ri] : ri];
    const size_t base = ((size_t)ri * nh + head) * n_splits;
    float M = -INFINITY, L = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < n_splits; s0 += GROUP) {
        float m[GROUP], l[GROUP];
        f32x4 o[GROUP];
#pragma unroll
        for (int i = 0; i < GROUP; ++i) {
            const int s = s0 + i < n_splits ? s0 + i : n_splits - 1;        // past the end: the last part again, weight 0
            m[i] = part_ml[(base + s) * 2];
            l[i] = part_ml[(base + s) * 2 + 1];
            o[i] = *(const f32x4 *)(part_o + (base + s) * DH + d0);
        }
        float Mn = M;
#pragma unroll
        for (int i = 0; i < GROUP; ++i) Mn = fmaxf(Mn, m[i]);
        const float M_safe = Mn == -INFINITY ? 0.f : Mn;
        const float keep = exp2f(M - M_safe);                                // 0 at the first group
        L *= keep;
        acc *= keep;
#pragma unroll
        for (int i = 0; i < GROUP; ++i) {
            const float f = s0 + i < n_splits ? exp2f(m[i] - M_safe) : 0.f;
            L += l[i] * f;
            acc += o[i] * f;
        }
        M = Mn;
    }
    const float inv = 1.0f / L;
    u32x2 w;
    w.x = pack_bf16(acc[0] * inv, acc[1] * inv);
    w.y = pack_bf16(acc[2] * inv, acc[3] * inv);
    *(u32x2 *)(out + (size_t)token * out_stride + (size_t)head * DH + d0) = w;
}

template <int DH>
static int launch_decode(const void *q, int q_stride, void *out, int out_stride, const void *cache,
                         const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                         const int *req_list, int n_req, int nh, int nkvh, int page, float scale, int window,
                         int n_splits, float *part_o, float *part_ml, hipStream_t stream) {
    const int g = nh / nkvh, chunks = (g + 15) / 16;
    const float scale_log2 = scale * 1.4426950408889634f;
    const size_t lds_bytes = (size_t)DEC_WAVES * 16 * (DH + 2) * sizeof(float);
    dim3 grid(n_req * nkvh * chunks, n_splits), block(DEC_WAVES * WAVE);
    // Two ways to address the pages (the same arithmetic, the same results).  FLAT: every lane holds
    // full addresses and reads the block table itself.  Not FLAT: the wave's number and with it the
    // pages are scalar, the loads are buffer loads with one lane offset for keys and one for values,
    // and the table is read a step ahead.  Measured on the Llama-3-8B shape, whole decode step: the
    // second is 1 % faster where a part is a few steps long (8 requests of 2k keys in 4 parts), the
    // first 2 % faster where a wave walks many steps (32 or 64 requests, one part each).
    const bool flat = n_splits == 1;
    (flat ? attention_decode_kernel<DH, true> : attention_decode_kernel<DH, false>)<<<grid, block, lds_bytes, stream>>>(
        (const bf16_t *)q, q_stride, (bf16_t *)out, out_stride, (const bf16_t *)cache, block_table, max_pages, q_start,
        ctx_len, req_list, nh, nkvh, page, scale_log2, window, n_splits, part_o, part_ml);
    LCU_LAUNCH_CHECK();
    if (n_splits > 1) {
        attention_merge_kernel<DH><<<dim3(n_req, nh), dim3(DH / 4), 0, stream>>>((bf16_t *)out, out_stride, part_o, part_ml,
                                                                                q_start, req_list, nh, n_splits);
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}

// The n_req requests req_list[0..n_req) of the batch (all of the batch's requests in order
// if req_list is null) feed exactly one token each.
// part_o: [n_req * nh * n_splits * dh] floats, part_ml: [n_req * nh * n_splits * 2] (unused
// when n_splits == 1).  bfloat16 only; head_dim 32, 64, 96 or 128; page_size a multiple of 16.
// What both decode entry points ask of their sizes (the parts' memory apart): LCU_OK or why not.
static int decode_arguments(int q_stride, int out_stride, int max_pages, int nh, int nkvh, int dh, int page, int window,
                            int n_splits) {
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || dh <= 0 || page <= 0 || page % 16 || max_pages <= 0 || window < 0 || n_splits < 1 ||
        n_splits > 65535 || q_stride % 8 || out_stride % 4)
        return LCU_BAD_ARGUMENT;
    if (dh != 32 && dh != 64 && dh != 96 && dh != 128) return LCU_UNSUPPORTED;
    if ((unsigned long long)kv_page_elems(nkvh, dh, page) * 2ull >= (1ull << 31)) return LCU_UNSUPPORTED;
    return LCU_OK;
}

LCU_API int lcu_attention_decode_bf16(const void *q, int q_stride, void *out, int out_stride, const void *cache,
                                      const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                                      const int *req_list, int n_req, int nh, int nkvh, int dh, int page, float scale,
                                      int window, int n_splits, float *part_o, float *part_ml, hipStream_t stream) {
    if (n_req <= 0) return LCU_OK;
    const int args = decode_arguments(q_stride, out_stride, max_pages, nh, nkvh, dh, page, window, n_splits);
    if (args != LCU_OK) return args;
    if (n_splits > 1 && (!part_o || !part_ml)) return LCU_BAD_ARGUMENT;
#define GO(D) return launch_decode<D>(q, q_stride, out, out_stride, cache, block_table, max_pages, q_start, ctx_len, req_list, n_req, nh, nkvh, page, scale, window, n_splits, part_o, part_ml, stream)
    if (dh == 128) GO(128);
    if (dh == 64) GO(64);
    if (dh == 96) GO(96);
    if (dh == 32) GO(32);
#undef GO
    return LCU_UNSUPPORTED;
}

// ---------------------------------------------------------------------------- no allocation
// The decode entry point for callers that cannot allocate (see attention_static.h): the parts'
// partial results go to a buffer in the library's own device image.  In host code `scratch` is
// only the symbol's stand-in; its address on a device is what hipGetSymbolAddress gives there.
static __device__ __align__(256) unsigned char scratch[LCU_ATTENTION_STATIC_SCRATCH_BYTES];

constexpr int STATIC_MAX_DEVICES = 64;
static void *scratch_on_device[STATIC_MAX_DEVICES];     // per device: each holds its own copy at its own address
static std::mutex scratch_lock;

// The buffer's address on the current device, looked up at the first call there.  LCU_OK, LCU_UNSUPPORTED
// (a device number beyond the table) or LCU_RUNTIME_ERROR (the runtime refused the look-up).
static int static_scratch(void **ptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return LCU_RUNTIME_ERROR;
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return LCU_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_on_device[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return LCU_RUNTIME_ERROR;
        scratch_on_device[dev] = p;
    }
    *ptr = scratch_on_device[dev];
    return LCU_OK;
}

LCU_API int lcu_attention_static_init(void) {
    void *p = nullptr;
    return static_scratch(&p);
}

LCU_API long long lcu_attention_static_scratch_bytes(void) { return (long long)LCU_ATTENTION_STATIC_SCRATCH_BYTES; }

LCU_API long long lcu_attention_static_scratch_needed(int n_req, int nh, int dh, int n_splits) {
    if (n_req <= 0 || nh <= 0 || dh <= 0 || n_splits <= 1) return 0;
    // sizes so large that the product leaves 63 bits need more than any buffer: the largest number says so
    const unsigned __int128 bytes = (unsigned __int128)n_req * (unsigned)nh * (unsigned)n_splits * (unsigned)(dh + 2) * sizeof(float);
    return bytes > (unsigned __int128)0x7fffffffffffffffll ? 0x7fffffffffffffffll : (long long)bytes;
}

LCU_API int lcu_attention_decode_bf16_static(const void *q, int q_stride, void *out, int out_stride, const void *cache,
                                             const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                                             const int *req_list, int n_req, int nh, int nkvh, int dh, int page, float scale,
                                             int window, int n_splits, hipStream_t stream) {
    if (n_req <= 0) return LCU_OK;
    // the arguments first, as the other entry point checks them: a call with bad sizes is told so, whatever
    // buffer it would need
    const int args = decode_arguments(q_stride, out_stride, max_pages, nh, nkvh, dh, page, window, n_splits);
    if (args != LCU_OK) return args;
    float *part_o = nullptr, *part_ml = nullptr;
    if (n_splits > 1) {
        if (lcu_attention_static_scratch_needed(n_req, nh, dh, n_splits) > (long long)LCU_ATTENTION_STATIC_SCRATCH_BYTES)
            return LCU_SCRATCH_EXCEEDED;
        void *base = nullptr;
        const int st = static_scratch(&base);
        if (st != LCU_OK) return st;
        part_o = (float *)base;                                            // [n_req * nh * n_splits * dh]
        part_ml = part_o + (size_t)n_req * nh * n_splits * dh;            // [n_req * nh * n_splits * 2]
    }
    return lcu_attention_decode_bf16(q, q_stride, out, out_stride, cache, block_table, max_pages, q_start, ctx_len, req_list,
                                     n_req, nh, nkvh, dh, page, scale, window, n_splits, part_o, part_ml, stream);
}

// ============================================================================ prefill
#ifndef LCU_PRE_MIN_WAVES
#define LCU_PRE_MIN_WAVES 2
#endif
constexpr int PRE_WAVES = 4;              // waves of a workgroup, each with 32 rows of its own: one wave per SIMD, so that a
                                          // compute unit holds two workgroups (two tasks) whose turns are not in step
constexpr int PRE_THREADS = PRE_WAVES * WAVE;
constexpr int PRE_RING = 3;               // buffers of 32 keys in LDS: one is read, two are on their way

// Wait until at most `left` of this wave's vector memory operations are outstanding.
template <int LEFT>
__device__ __forceinline__ void wait_loads() {
    static_assert(LEFT >= 0 && LEFT < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt((LEFT & 15) | ((LEFT >> 4) << 14) | (7 << 4) | (15 << 8));
}

// The prefill kernel's arithmetic on v_mfma_f32_32x32x16_bf16.  A wave holds 32 rows (lane % 32 is the
// row, both for Q as the B operand and for S^T and O^T as results), so every lane owns ONE row: its
// 16 scores of a step of 32 keys lie in its own registers, the row's maximum crosses lanes once
// (lane and lane + 32), and maximum, sum and rescaling are kept once per lane.
//   S^T[key, row] = K[key, :] . Q[row, :]     A = K: lane holds 8 dims (16 sidx + 8 hi ..) of the key in
//                                             slot lane % 32: one 16-byte read of the keys' copy in LDS
//   O^T[dim, row] += V^T[dim, key] . P^T[key, row]   A = V^T: lane holds 8 keys of dim 32 t + lane % 32,
//                                             B = P^T: the lane's own scores
// Result element i of a lane (hi = lane / 32) is row 8 (i / 4) + 4 hi + i % 4 of the instruction.  The
// keys' copy in LDS stands so (stage_issue) that row m of the first product is key
// 16 (m / 16) + (m % 16 with bits 2 and 3 swapped) of the step: a lane's elements 8 kk .. 8 kk + 7 are then
// the keys 16 kk + 8 hi .. + 7 in a row, which is what its 16-byte read of the values' copy holds.
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <int DH>
struct PrefillState {
    f32x16 o[DH / 32];      // O^T: lane = (row lane % 32, dims 32 t + 8 (i / 4) + 4 hi + i % 4)
    float m;                // running maximum (in units of log2), the same in the row's two lanes
    float l;                // running sum over the lane's own keys only
};

// The larger of the values that lane l and lane l ^ 32 hold, in both.
__device__ __forceinline__ float max_over_halves(float x) {
    const unsigned u = __float_as_uint(x);
    const auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// The keys and values of a step of 32 keys, copied into LDS in chunks of 16 bytes: 8 * DH
// chunks, [K tile 0 | K tile 1 | V tile 0 | V tile 1], 2 * DH chunks per tile of 16 keys.  Keys as the page
// holds them, [dim / 8][slot 16], the token in slot p being p with bits 2 and 3 swapped.  Values: [half][dim], the chunk of tokens 8 half .. + 7 of the tile for every dim (the page holds
// [dim][token]).  With these orders the lanes of every read of an operand take neighbouring bytes: no bank
// conflicts (with the values as their page has them four lanes of a read fell into one bank, and the
// conflicts took a quarter of the kernel's time).  A thread of the workgroup copies chunks tid, tid + 256, ...
//
// The copy goes from memory straight into LDS (buffer_load ... lds: no registers hold the data on its way,
// lane l of a wave writes the 16 bytes l of the wave's 1 KB), so the loads of two buffers can be in flight
// while one is computed.  Everything but the lane's offset is made in scalar registers from the wave's
// number: a wave's 64 chunks lie in one region of one step (regions are multiples of 64 chunks), and a
// tile of 16 keys lies in one page, whose number is read through the scalar unit (which does not make
// the wave wait for the vector loads in flight); the buffer of the load is the page.  Tile T is in page
// T / (page / 16): with tile_magic = floor(2^32 / (page / 16)) + 1 the quotient is the high word of
// T * tile_magic (exact while T * page / 16 < 2^32; 0 stands for pages of 16 keys, where the page is the
// tile).  Steps beyond the end of the keys are copied all the same, from the pages that the clamped block
// table names (valid memory), into a buffer that nobody reads: no branch around a load.  A page holds
// less than 2 GiB (the host checks).
// What a lane adds to the scalar part of its chunks' addresses: the same in every step, so it is made
// once per task and kept (one register for the keys, one per load for the values).
template <int DH>
struct StageLane {
    uint32_t k;               // keys: a wave holds 4 dim chunks x 16 slots
    uint32_t v[DH / 32];      // values: the lane's chunk is number w0 + lane of [half][dim] (a wave may hold the end of
                              // one half and the start of the other where head_dim is no multiple of 64)
};

template <int DH>
__device__ __forceinline__ void stage_lane(StageLane<DH> &sl, int page, int wave_id, int lane) {
    constexpr uint32_t E = sizeof(bf16_t);
    const uint32_t k_tok = (lane & 3) | ((lane & 4) << 1) | ((lane & 8) >> 1);
    sl.k = ((uint32_t)(lane >> 4) * page + k_tok) * 8 * E;
#pragma unroll
    for (int i = 0; i < DH / 32; ++i) {
        const int w0 = (wave_id * WAVE + PRE_THREADS * i) % (2 * DH);
        const uint32_t v_at = (uint32_t)(w0 + lane), v_half = v_at / DH, v_dim = v_at - v_half * DH;
        sl.v[i] = (v_dim * page + 8 * v_half) * E;
    }
}

// The pages of the wave's chunks of a copy (through the scalar unit), and each chunk's first token in its
// page: the keys of the step at kk0 and the values of the step at vk0 (the keys run two steps ahead of the
// values, see the kernel).  Read one turn before the copy that uses them, so that the
// copy does not wait for the table.
template <int DH, bool PAGE16>
__device__ __forceinline__ void stage_pages(int *page_id, uint32_t *tok0, const int *__restrict__ bt,
                                            int max_pages, int page, uint32_t tile_magic, int kk0, int vk0, int wave_id) {
    const int tiles_per_page = page / 16;
#pragma unroll
    for (int i = 0; i < DH / 32; ++i) {
        const int cw = wave_id * WAVE + PRE_THREADS * i;          // the wave's first chunk
        const int region = cw / (2 * DH), t = region & 1;
        const uint32_t tile = (uint32_t)((region < 2 ? kk0 : vk0) >> 4) + t;
        int pi = (int)tile;                                       // pages of 16 keys: the page is the tile
        tok0[i] = 0;
        if (!PAGE16) {
            pi = (int)__umulhi(tile, tile_magic);
            tok0[i] = (tile - (uint32_t)pi * tiles_per_page) * 16;
        }
        pi = pi < max_pages ? pi : max_pages - 1;
        page_id[i] = bt[pi];
    }
}

// FLAT: the whole cache of the layer is one buffer of less than 4 GiB (the host says), and a page is an
// offset in it: two scalar instructions per chunk.  Else the buffer of a load is its page, whose 64-bit
// address is made per chunk (a dozen scalar instructions: with four chunks a step they were a third
// of all the instructions a wave issued).
template <int DH>
__device__ __forceinline__ void stage_issue(u32x4 *__restrict__ buf, const bf16_t *__restrict__ cache, bool FLAT,
                                            uint32_t cache_bytes, const int *page_id,
                                            const uint32_t *tok0, const StageLane<DH> &sl, int page, size_t page_elems,
                                            int nkvh, int kvh, int wave_id) {
    constexpr uint32_t E = sizeof(bf16_t);
#pragma unroll
    for (int i = 0; i < DH / 32; ++i) {
        const int cw = wave_id * WAVE + PRE_THREADS * i;          // the wave's first chunk
        const int region = cw / (2 * DH), w0 = cw % (2 * DH);
        // keys: dim chunks w0 / 16 .. + 3 of the tile
        const uint32_t s_off = region < 2 ? ((uint32_t)(kvh * (DH / 8) + w0 / 16) * page + tok0[i]) * 8 * E
                                          : ((uint32_t)((nkvh + kvh) * DH) * page + tok0[i]) * E;
        // (a plain variable: the compiler's pass for the host refuses the load builtin with an argument whose
        // type depends on a template parameter)
        const uint32_t lane_off = region < 2 ? sl.k : sl.v[i];
        if (FLAT) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(cache), 0, cache_bytes, 0x00020000),
                (__attribute__((address_space(3))) void *)(buf + cw), 16, lane_off,
                (uint32_t)page_id[i] * (uint32_t)(page_elems * E) + s_off, 0, 0);
        } else {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(cache + (size_t)page_id[i] * page_elems), 0,
                                                  (uint32_t)(page_elems * E), 0x00020000),
                (__attribute__((address_space(3))) void *)(buf + cw), 16, lane_off,
                s_off, 0, 0);
        }
    }
}

// Where a lane's keys (for the scores) and values (for the output) of a step's copy stand in LDS.
// values: dim 32 t + n, keys 16 kk + 8 hi .. + 7: V tile kk, half hi; chunk kk * 2 DH + 32 t from there
// keys: row m = n of the instruction: key tile n / 16, slot n % 16; dims 16 sidx + 8 hi ..: dim chunk 2 sidx + hi;
// chunk 32 sidx from there
template <int DH>
__device__ __forceinline__ const u32x4 *lane_values(const u32x4 *buf, int n, int hi) { return buf + 4 * DH + hi * DH + n; }
template <int DH>
__device__ __forceinline__ const u32x4 *lane_keys(const u32x4 *buf, int n, int hi) { return buf + (n >> 4) * 2 * DH + hi * 16 + (n & 15); }

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant in its body.
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

// Chunk CHUNK behind `from` in LDS into the registers of `r`: an ordinary load, which the compiler waits for where the
// register is used, by its own count.  The fence keeps the load where it stands, behind the instruction that used the
// register's old contents: the old and the new value then never live at once, and the register allocator gives both
// the same register (without the fence the scheduler read all keys early into new registers and copied them over at
// the end of every turn, 24 copies a turn).  `from` is derived from a __restrict__ parameter of the function that also
// issues the copies into LDS, so the read does not wait for them (through an integer address the compiler put a wait
// for every copy in flight before the reads).
template <int CHUNK>
__device__ __forceinline__ void lds_read_plain(u32x4 &r, const u32x4 *from) {
    r = from[CHUNK];
    __builtin_amdgcn_sched_barrier(0);
}

// Nothing that uses the operands read so far moves above this point, and nothing that stands above moves below.
__device__ __forceinline__ void operands_fence() { __builtin_amdgcn_sched_barrier(0); }

// One turn of a wave: the output of step e - 1 and the scores and the softmax of step e, 32 keys each, for
// the wave's 32 rows.
//   output   O += V(e - 1)^T P(e - 1)     `v` and `pb` as the turn before has left them
//   scores   S(e) = K(e) Q^T              `k` as the turn before has left it
//   softmax  P(e) from S(e)               into `pb`; then O goes over to the new reference point
// The keys are in registers when the turn begins (the turn before has read them from LDS).  The turn reads
// the values V(e - 1) into the registers that the turn before has used up, first of all, so that they arrive
// during the scores' matrix instructions, and the keys of the next turn, K(e + 1), each into the registers of
// the keys that a matrix instruction has just used, so that they arrive during the softmax (both from `next`:
// 8 * DH chunks).  The output's matrix instructions and the softmax need nothing of each other and stand in
// one block: the vector unit works while the matrix cores do (a matrix instruction takes 8 passes; about 7
// vector instructions fit beside it; with the stages one after the other the two units took turns).
//
// It also issues a copy into `dst`, a buffer of the ring other than `next`, which the qualifiers of the two
// pointers say: both must be parameters of ONE function for that (the compiler knows nothing about two
// pointers that are parameters of different functions, or local variables, and then makes every read from
// LDS wait for every copy in flight, which empties the ring of copies in every turn).
//
// k0: the first key of step e; p_row / lo_row: the last and first key that the lane's row may see; mask (the
// same in the whole wave): some row does not see all 32 keys of step e.  A step that is none of the wave's
// comes with mask and p_row = -1: all its weights are zero and nothing changes.  maskv, p_max / lo_min: the
// same for the values of step e - 1: values of keys that no row of the wave sees are taken as zero,
// whatever the memory holds (all of them with p_max = -1).
//
// There is one body for masked and unmasked steps, and everything that changes the output in it works
// in place (the matrix instructions add to their own operand, the rescaling and the clearing of unseen
// values are written as instructions on their own registers).  With a body for each case, or with the
// rescaling as plain arithmetic under its branch, the compiler kept the 64 registers of the output in
// one place across the loop and in another inside it, and copied them both ways in every step: more
// instructions than the softmax itself.
template <int DH, class Issue, class Pages>
__device__ __forceinline__ void attn_turn(const u32x4 *__restrict__ next, u32x4 *__restrict__ dst, Issue &&issue_copy, Pages &&ask_pages,
                                          u32x4 (&k)[DH / 16], u32x4 (&v)[2 * (DH / 32)], u32x4 (&pb)[2], const u32x4 (&q)[DH / 16],
                                          PrefillState<DH> &st, float &alpha, int k0, bool mask, int p_row, int lo_row, bool maskv,
                                          int p_max, int lo_min, float scale_log2, int n, int hi) {
    issue_copy(dst);
    // the values of step e - 1: on their way during the scores' matrix instructions (they stand before the
    // branch below, in a block of their own: in one block with the matrix instructions the compiler's
    // scheduler put them behind most of those, and the wait for them was 5 % of the kernel's time)
    const u32x4 *ka = lane_keys<DH>(next, n, hi), *va = lane_values<DH>(next, n, hi);
    static_for<2 * (DH / 32)>([&](auto i) {
        constexpr int kk = decltype(i)::value / (DH / 32), t = decltype(i)::value % (DH / 32);
        lds_read_plain<kk * 2 * DH + 32 * t>(v[decltype(i)::value], va);
    });
    // the output so far goes over to the reference point that the turn before has chosen (here, and not where
    // that turn made the factor: a branch behind the softmax would cut it off the block of the matrix
    // instructions)
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int t = 0; t < DH / 32; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(st.o[t][i]) : "v"(alpha));
    }
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    static_for<DH / 16>([&](auto i) {
        constexpr int sidx = decltype(i)::value;
        s = mfma32(k[sidx], q[sidx], s);
        lds_read_plain<32 * sidx>(k[sidx], ka);                    // the keys of step e + 1
    });
    operands_fence();
    ask_pages();                                   // (scalar loads: behind the matrix instructions and the reads from LDS)
    if (maskv) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            uint32_t keep[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int j = k0 - 32 + 16 * kk + 8 * hi + e;
                if (j > p_max || j < lo_min) keep[e / 2] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
            }
#pragma unroll
            for (int t = 0; t < DH / 32; ++t) {
                asm volatile("v_and_b32 %0, %0, %1" : "+v"(v[kk * (DH / 32) + t].x) : "v"(keep[0]));
                asm volatile("v_and_b32 %0, %0, %1" : "+v"(v[kk * (DH / 32) + t].y) : "v"(keep[1]));
                asm volatile("v_and_b32 %0, %0, %1" : "+v"(v[kk * (DH / 32) + t].z) : "v"(keep[2]));
                asm volatile("v_and_b32 %0, %0, %1" : "+v"(v[kk * (DH / 32) + t].w) : "v"(keep[3]));
            }
        }
    }
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = s[i];
    if (mask) {
        // a lane's score i is key k0 + 8 hi + c with c = 16 (i / 8) + i % 8: compared as c against the bounds less k0 + 8 hi
        const int last = p_row - k0 - 8 * hi, first = lo_row - k0 - 8 * hi;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = 16 * (i / 8) + i % 8;
            if (c > last || c < first) x[i] = -INFINITY;
        }
    }
    // the keys of the next turn: here rather than at the turn's end (it costs nothing: the other workgroup's
    // waves have work), so that the long block below, where registers are scarce, is outside the stretch
    // in which the keys' registers may not be touched
    operands_fence();
    // the output's matrix instructions stand here, beside the softmax that does not need them: the
    // compiler's scheduler puts vector instructions between them (its own mix was the fastest: with ten
    // vector instructions forced behind each matrix instruction the kernel was 11 % slower, with all the
    // matrix instructions first 4 %)
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int t = 0; t < DH / 32; ++t) st.o[t] = mfma32(v[kk * (DH / 32) + t], pb[kk], st.o[t]);
    float mx = fmaxf(fmaxf(x[0], x[1]), x[2]);
#pragma unroll
    for (int i = 3; i < 15; i += 2) mx = fmaxf(fmaxf(mx, x[i]), x[i + 1]);
    mx = fmaxf(mx, x[15]);
    mx = max_over_halves(mx);
    // the reference point of the exponentials moves only when the maximum has grown by more than
    // 2^RESCALE_SLACK: the weights stay below that, and the output is rarely rescaled
    const float m_true = fmaxf(st.m, mx * scale_log2);
    const float m_new = m_true - st.m <= RESCALE_SLACK ? st.m : m_true;       // false for the first keys (-inf)
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    alpha = fast_exp2(st.m - m_safe);              // for the output, the values of step e - 1 included: in the next turn
    float p[16], sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] = fast_exp2(fmaf(x[i], scale_log2, -m_safe));
        sum += p[i];
    }
    st.l = st.l * alpha + sum;
    st.m = m_new;
    u32x4 pb_new[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
        pb_new[kk] = u32x4{pack_bf16(p[8 * kk], p[8 * kk + 1]), pack_bf16(p[8 * kk + 2], p[8 * kk + 3]),
                           pack_bf16(p[8 * kk + 4], p[8 * kk + 5]), pack_bf16(p[8 * kk + 6], p[8 * kk + 7])};
    pb[0] = pb_new[0];
    pb[1] = pb_new[1];
}

// A task is a block of consecutive tokens of one request: a workgroup has 4 waves, one per SIMD; each takes
// 32 rows (tokens x the heads of one chunk of a group), so a task covers 4 * (32 / heads per chunk) tokens,
// starting at batch index task_tok0[t].  The workgroup walks the keys that any of its rows sees, 32 at a
// time; the keys and values are copied to LDS once per workgroup, two buffers ahead of the one that is
// read: before a turn every wave waits for its own part of a copy, then a barrier (which waits for LDS
// only) makes the whole copy visible and says that the buffer of the turn before is free for the copy two
// ahead.  A compute unit holds two workgroups (48 KB of LDS and half the registers each), so every SIMD has
// two waves of two different tasks: their turns are not in step (while one wave's softmax keeps the vector
// unit busy the other's matrix instructions run), and what a task costs before its first and after its last
// turn (its tables, its queries, the first copy: some microseconds of waiting for memory) the other task
// fills.  (Eight waves that worked on one task, in two halves that split the keys and met at a barrier every
// turn, were as fast over long contexts and a tenth slower where tasks are short: portions of 256 tokens over
// 2k keys 83 against 75 us, a single task of 32 tokens 11.9 against 8.8 us.)
template <int DH, bool PAGE16, bool FLAT>
__global__ void __launch_bounds__(PRE_THREADS, LCU_PRE_MIN_WAVES)
attention_prefill_kernel(const bf16_t *__restrict__ q, int q_stride, bf16_t *__restrict__ out, int out_stride,
                           const bf16_t *__restrict__ cache, uint32_t cache_bytes, const int *__restrict__ block_table, int max_pages,
                           const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                           const int *__restrict__ task_req, const int *__restrict__ task_tok0, int max_tasks,
                           const int *__restrict__ n_tasks_dev,
                           int tasks_per_wg, int nh, int nkvh, int page, uint32_t tile_magic, float scale_log2, int window) {
    extern __shared__ u32x4 lds_ring[];            // [PRE_RING][8 * DH]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int lane = threadIdx.x & (WAVE - 1);
    // Workgroups go to the chip's eight dies in turn (workgroup i to die i % 8), and each die has an L2 of
    // its own.  The key/value head is the fastest index of the grid, so that the workgroups of one head
    // (with 8 heads, or a multiple or a divisor of 8) all run on one die, whose L2 then holds that head's keys and
    // values for all of them: with the task as the fastest index every die read every head's keys.
    const int g = nh / nkvh;
    const int chunks = (g + 15) / 16;
    const int head_chunk = blockIdx.x % (nkvh * chunks), wg = blockIdx.x / (nkvh * chunks);
    // the grid is made for max_tasks; how many of them the list holds may stand in memory (so that a launch recorded
    // into a graph serves steps with other lists): workgroups beyond the list's end have nothing to do
    const int n_tasks = n_tasks_dev ? min(*n_tasks_dev, max_tasks) : max_tasks;
    for (int task = wg * tasks_per_wg; task < (wg + 1) * tasks_per_wg && task < n_tasks; ++task) {
    __syncthreads();                               // the last task's use of LDS is over (it waited for its copies)
    const int n = lane & 31, hi = lane >> 5;
    const int kvh = head_chunk / chunks, chunk = head_chunk % chunks;
    const int hc = (g - 16 * chunk) < 16 ? (g - 16 * chunk) : 16;      // heads of this chunk
    const int tokens_per_wave = 32 / hc;                                // tokens in 32 rows
    const int r = task_req[task], task_tok = task_tok0[task];
    const int q_end = q_start[r + 1];
    const int ctx = ctx_len[r];
    const int head0 = kvh * g + 16 * chunk;
    const int tok0 = task_tok + wave * tokens_per_wave;                 // this wave's first token
    const int pos_of_tok = ctx - q_end;                                 // a token's position = its batch index + this

    const int tok = tok0 + n / hc;
    const bool valid = n < tokens_per_wave * hc && tok < q_end;
    const int tok_row = valid ? tok : -1;
    u32x4 qv[DH / 16];
    {
        const bf16_t *qrow = q + (size_t)(valid ? tok : task_tok) * q_stride + (size_t)(head0 + n % hc) * DH;
#pragma unroll
        for (int sidx = 0; sidx < DH / 16; ++sidx)
            qv[sidx] = valid ? *(const u32x4 *)(qrow + 16 * sidx + 8 * hi) : u32x4{0u, 0u, 0u, 0u};
    }
    // what this wave sees (the same in all its lanes), and what the workgroup sees
    const bool wave_has = tok0 < q_end;
    int p_max = -1, p_min = -1, lo_min = 0, lo_max = 0;
    if (wave_has) {
        const int last_tok = (tok0 + tokens_per_wave < q_end ? tok0 + tokens_per_wave : q_end) - 1;
        p_max = ctx - (q_end - last_tok);
        p_min = ctx - (q_end - tok0);
        lo_min = window > 0 && p_min - window + 1 > 0 ? p_min - window + 1 : 0;
        lo_max = window > 0 && p_max - window + 1 > 0 ? p_max - window + 1 : 0;
    }
    const int wg_last_tok = (task_tok + PRE_WAVES * tokens_per_wave < q_end ? task_tok + PRE_WAVES * tokens_per_wave : q_end) - 1;
    const int wg_p_max = ctx - (q_end - wg_last_tok);
    const int wg_p_min = ctx - (q_end - task_tok);
    const int wg_lo_min = window > 0 && wg_p_min - window + 1 > 0 ? wg_p_min - window + 1 : 0;

    PrefillState<DH> st;
    st.m = -INFINITY;
    st.l = 0.f;
#pragma unroll
    for (int t = 0; t < DH / 32; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) st.o[t][i] = 0.f;
    const int *bt = block_table + (size_t)r * max_pages;
    const size_t page_elems = kv_page_elems(nkvh, DH, page);
    const int blk0 = wg_lo_min / 32, n_steps = wg_p_max / 32 + 1 - blk0;
    StageLane<DH> sl;
    stage_lane<DH>(sl, page, wave, lane);
    int page_id[DH / 32];
    uint32_t tok_in_page[DH / 32];
    // Copy c holds the keys of step c and the values of step c - 2 (of step 0 where there is none: nobody
    // uses them): what turn c - 1 of a wave reads into its registers.  Copy e + 3 is issued in turn e, into
    // the buffer of copy e.
    auto keys_from = [&](int c) { return (blk0 + c) * 32; };
    auto values_from = [&](int c) { return (blk0 + (c > 1 ? c - 2 : 0)) * 32; };
#pragma unroll
    for (int c = 0; c < PRE_RING; ++c) {
        stage_pages<DH, PAGE16>(page_id, tok_in_page, bt, max_pages, page, tile_magic, keys_from(c), values_from(c), wave);
        stage_issue<DH>(lds_ring + c * 8 * DH, cache, FLAT, cache_bytes, page_id, tok_in_page, sl, page, page_elems, nkvh, kvh, wave);
    }
    stage_pages<DH, PAGE16>(page_id, tok_in_page, bt, max_pages, page, tile_magic, keys_from(PRE_RING), values_from(PRE_RING), wave);
    const int p_row = tok_row < 0 ? -1 : tok_row + pos_of_tok;
    const int lo_row = tok_row >= 0 && window > 0 && p_row - window + 1 > 0 ? p_row - window + 1 : 0;
    u32x4 kreg[DH / 16], vreg[2 * (DH / 32)];
    u32x4 pb[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
    wait_loads<(PRE_RING - 1) * (DH / 32)>();
    lds_barrier();
    {
        const u32x4 *kb = lane_keys<DH>(lds_ring, n, hi);
#pragma unroll
        for (int sidx = 0; sidx < DH / 16; ++sidx) kreg[sidx] = kb[32 * sidx];
#pragma unroll
        for (int i = 0; i < 2 * (DH / 32); ++i) vreg[i] = u32x4{0u, 0u, 0u, 0u};
    }
    int slot = 1, fill = 0;                       // the buffers of copy e + 1 and of copy e
    bool own_before = false, mask_before = true;      // the first turn's values are nobody's: all taken as zero
    float alpha = 1.0f;
    for (int e = 0; e < n_steps + 1; ++e) {
        // copy e + 1 has landed (this wave's part of it; the barrier says so for the others'), and every wave
        // has read copy e (a turn ends with its reads from LDS over)
        wait_loads<(PRE_RING - 2) * (DH / 32)>();
        lds_barrier();
        // the copy into the freed buffer uses the pages read a turn ago; then the pages of the copy after that
        // one are asked for, there when the next turn needs them
        int page_now[DH / 32];
        uint32_t tok_now[DH / 32];
#pragma unroll
        for (int i = 0; i < DH / 32; ++i) page_now[i] = page_id[i], tok_now[i] = tok_in_page[i];
        auto issue_copy = [&](u32x4 *__restrict__ to) {
            stage_issue<DH>(to, cache, FLAT, cache_bytes, page_now, tok_now, sl, page, page_elems, nkvh, kvh, wave);
        };
        auto ask_pages = [&]() {
            stage_pages<DH, PAGE16>(page_id, tok_in_page, bt, max_pages, page, tile_magic, keys_from(e + PRE_RING + 1), values_from(e + PRE_RING + 1), wave);
        };
        // is step e one of the wave's, and does some row not see all its keys?  (the same of step e - 1, for
        // its values, from the turn before)
        const int k0 = (blk0 + e) * 32;
        const bool own = e < n_steps && wave_has && k0 <= p_max && k0 + 31 >= lo_min;
        const bool mask = !own || k0 + 31 > p_min || k0 < lo_max;
        attn_turn<DH>(lds_ring + slot * 8 * DH, lds_ring + fill * 8 * DH, issue_copy, ask_pages, kreg, vreg, pb, qv, st,
                      alpha, k0, mask, own ? p_row : -1, lo_row, mask_before, own_before ? p_max : -1, lo_min, scale_log2, n, hi);
        own_before = own;
        mask_before = mask;
        slot = slot + 1 == PRE_RING ? 0 : slot + 1;
        fill = fill + 1 == PRE_RING ? 0 : fill + 1;
    }
    wait_loads<0>();                               // the last copies into the ring, which nobody reads, have landed
    // ---- a row's sum lies in its two lanes (each added the keys it held); the output is written as it stands
    float l_all = st.l;
    l_all += __shfl_xor(l_all, 32, WAVE);
    const float inv = 1.0f / l_all;
    if (tok_row >= 0) {
        bf16_t *o = out + (size_t)tok_row * out_stride + (size_t)(head0 + n % hc) * DH;
#pragma unroll
        for (int t = 0; t < DH / 32; ++t)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                u32x2 w;
                w.x = pack_bf16(st.o[t][4 * b] * inv, st.o[t][4 * b + 1] * inv);
                w.y = pack_bf16(st.o[t][4 * b + 2] * inv, st.o[t][4 * b + 3] * inv);
                *(u32x2 *)(o + 32 * t + 8 * b + 4 * hi) = w;
            }
    }
    }
}

template <int DH, bool PAGE16, bool FLAT>
static int launch_prefill_as(const void *q, int q_stride, void *out, int out_stride, const void *cache, uint32_t cache_bytes,
                             const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                             const int *task_req, const int *task_tok0, int n_tasks, const int *n_tasks_dev, int tasks_per_wg,
                             int nh, int nkvh, int page, float scale, int window, hipStream_t stream) {
    const int g = nh / nkvh, chunks = (g + 15) / 16;
    const long long n_wg = (long long)((n_tasks + tasks_per_wg - 1) / tasks_per_wg) * nkvh * chunks;
    if (n_wg > 0x7fffffffll) return LCU_BAD_ARGUMENT;
    dim3 grid((unsigned)n_wg), block(PRE_THREADS);
    constexpr size_t lds_bytes = (size_t)PRE_RING * 8 * DH * sizeof(u32x4);
    // more than 64 KB of LDS must be asked for once, on every device that runs the kernel
    static std::mutex lock;
    static bool allowed[STATIC_MAX_DEVICES] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) return LCU_RUNTIME_ERROR;
    {
        std::lock_guard<std::mutex> guard(lock);
        if (!allowed[dev]) {
            const hipError_t e = hipFuncSetAttribute((const void *)attention_prefill_kernel<DH, PAGE16, FLAT>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return (int)e;
            allowed[dev] = true;
        }
    }
    attention_prefill_kernel<DH, PAGE16, FLAT><<<grid, block, lds_bytes, stream>>>(
        (const bf16_t *)q, q_stride, (bf16_t *)out, out_stride, (const bf16_t *)cache, cache_bytes, block_table, max_pages, q_start,
        ctx_len, task_req, task_tok0, n_tasks, n_tasks_dev, tasks_per_wg, nh, nkvh, page,
        page == 16 ? 0u : (uint32_t)(0x100000000ull / (unsigned)(page / 16)) + 1u, scale * 1.4426950408889634f, window);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// cache_pages: the number of pages of the layer's cache (its size decides how pages are addressed).
template <int DH>
static int launch_prefill(const void *q, int q_stride, void *out, int out_stride, const void *cache, long long cache_pages,
                          const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                          const int *task_req, const int *task_tok0, int n_tasks, const int *n_tasks_dev, int tasks_per_wg,
                          int nh, int nkvh, int page, float scale, int window, hipStream_t stream) {
    const unsigned long long bytes = (unsigned long long)cache_pages * kv_page_elems(nkvh, DH, page) * sizeof(bf16_t);
    const bool flat = bytes < (1ull << 32);
#define AS(P, F) return launch_prefill_as<DH, P, F>(q, q_stride, out, out_stride, cache, (uint32_t)(F ? bytes : 0), block_table, max_pages, q_start, ctx_len, task_req, task_tok0, n_tasks, n_tasks_dev, tasks_per_wg, nh, nkvh, page, scale, window, stream)
    if (page == 16) {
        if (flat) AS(true, true);
        AS(true, false);
    }
    if (flat) AS(false, true);
    AS(false, false);
#undef AS
}

// How many consecutive tokens of one request a task of the prefill kernel covers, for a
// model with `nh` heads in `nkvh` groups (the host cuts the batch into tasks with it).
LCU_API int lcu_attention_prefill_tokens_per_task(int nh, int nkvh) {
    if (nh <= 0 || nkvh <= 0 || nh % nkvh) return 0;
    const int g = nh / nkvh;
    if (g > 16 && g % 16) return 0;       // chunks of a group must be equal for one task size
    const int hc = g < 16 ? g : 16;
    return PRE_WAVES * (32 / hc);
}

// task_req / task_tok0: [n_tasks], tasks cut from the batch with the size above; a
// request's last task may be shorter.  Workgroup i takes tasks i*tasks_per_wg .. + tasks_per_wg-1.
// n_tasks_dev (may be null): a number on the device, read when the kernel runs: the lists hold that many tasks
// (at most n_tasks, for which the grid is made), so that one recorded launch serves lists of other lengths.
// bfloat16 only; head_dim 32, 64, 96 or 128; page_size a multiple of 16.
LCU_API int lcu_attention_prefill_bf16(const void *q, int q_stride, void *out, int out_stride, const void *cache,
                                       long long cache_pages, const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                                       const int *task_req, const int *task_tok0, int n_tasks, const int *n_tasks_dev,
                                       int tasks_per_wg, int nh, int nkvh, int dh, int page, float scale, int window,
                                       hipStream_t stream) {
    if (n_tasks <= 0) return LCU_OK;
    if ((unsigned long long)kv_page_elems(nkvh, dh, page) * 2ull >= (1ull << 31)) return LCU_UNSUPPORTED;
    if (cache_pages <= 0 || tasks_per_wg < 1 || lcu_attention_prefill_tokens_per_task(nh, nkvh) == 0 || page <= 0 || page % 16 || max_pages <= 0 ||
        window < 0 || q_stride % 8 || out_stride % 4 || nkvh * ((nh / nkvh + 15) / 16) > 65535)
        return LCU_BAD_ARGUMENT;
#define GO(D) return launch_prefill<D>(q, q_stride, out, out_stride, cache, cache_pages, block_table, max_pages, q_start, ctx_len, task_req, task_tok0, n_tasks, n_tasks_dev, tasks_per_wg, nh, nkvh, page, scale, window, stream)
    if (dh == 128) GO(128);
    if (dh == 64) GO(64);
    if (dh == 96) GO(96);
    if (dh == 32) GO(32);
#undef GO
    return LCU_UNSUPPORTED;
}
