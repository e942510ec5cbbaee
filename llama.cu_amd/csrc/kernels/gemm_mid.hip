// Y[M, N] = X[M, K] * W[N, K]^T for 17 to 256 rows (decoding many requests), bfloat16 operands,
// 32-bit accumulation on the matrix cores.  W is streamed once from HBM; what sets this kernel
// apart from the one for few rows is where X comes from.  With 64 rows a wave that loads its own
// piece of X moves twice as many bytes of X as of W and has no registers left to keep loads of W
// in flight.  Here
//
//   * a workgroup is four consumer waves (two for SwiGLU with up to 32 rows) and one producer
//     wave for every 64 rows.  The consumers work on the same k at the same time, each on its
//     own tile of 16 output features (for SwiGLU a gate tile and the up tile that belongs to
//     it), so one piece of X serves all of them;
//   * the producer wave does nothing but copy X, macro-step (128 k) by macro-step, from memory
//     (it comes from the L2 cache) into a ring of three buffers in LDS, two macro-steps ahead
//     (beyond 128 rows two buffers, one macro-step ahead: 256 rows fit twice into the 160 KB).
//     Its waits for its loads do not touch the consumers' loads: a wave's loads come back in
//     order, so a consumer that waited for X would wait for every load of W issued before it;
//   * a consumer keeps the loads of W of several macro-steps in flight (16 registers a tile and step),
//     reads X as matrix operands from LDS (rows 272 bytes apart: the 16 lanes of a read fall
//     into different banks) and multiplies: v_mfma_f32_16x16x32_bf16, A = W tile, B = X^T;
//   * a product with few output features is cut over K into slices (grid.y), so that the whole
//     chip streams W: each slice writes its partial sums as float32 to its own plane of the
//     output, [slice][M][N], and the kernel that follows (residual sum and norm) adds the planes
//     in a fixed order.  Nothing is added atomically: results do not depend on timing.
//
// A second kernel (gemm_mid_qkv_kernel, below) is the q, k, v product with the rotation and the cache write
// in its epilogue: there the consumer waves share each macro-step of K instead of the features.
//
// W is plain rows or packed as gemm_skinny.hip describes it (16 x 128 blocks of 4 KB).  (The reference
// gives every product to its vendor library, llama.cu/src/op/linear.rs:91-118; at these row counts the
// library streams the weights at half of what HBM gives.)
//
// The rows of X may wait for their normalisation (sumsq_in not null: a factor per row,
// rsqrt(sum of the row's shares / norm_width + eps), which commutes with the product): consumer
// wave w loads the shares of rows 16 w .. 16 w + 15 before its first loads of W, so they are back
// first, adds them in a fixed order and leaves the factors in LDS for the epilogue.
#include "common.h"
#include "kv_layout.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

enum { MID_EPI_BF16 = 0, MID_EPI_PARTIAL_F32 = 1, MID_EPI_SWIGLU = 2 };

#ifndef LCU_MID_STAGES
#define LCU_MID_STAGES 8
#endif
constexpr int MID_STAGE_TILES = LCU_MID_STAGES;    // tiles of W in flight per wave: stages times tiles of a wave
#ifndef LCU_MID_CONSUMERS
#define LCU_MID_CONSUMERS 4
#endif
constexpr int MID_CONSUMERS = LCU_MID_CONSUMERS;
#ifndef LCU_MID_XDEPTH
#define LCU_MID_XDEPTH 2                      // macro-steps of X that a producer has on their way in registers (twice as many for up to 32 rows)
#endif
constexpr int MID_STREAM = 2;                 // the loads of a packed W are non-temporal (read once; see gemm_skinny.hip's stream_load)
constexpr int MID_XROW = 272;                 // bytes between the rows of X in LDS (256 + 16)
constexpr int mid_xbufs(int MT) { return MT > 8 ? 2 : 3; }      // buffers of the ring of X (160 KB of LDS: 256 rows fit twice)

__device__ __forceinline__ f32x4 mid_mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

constexpr int mid_producers(int MT) { return (MT + 3) / 4; }
// Whether the loops run whole turns of their rings without a test of the step (below); beyond 192 rows, where the
// sums leave few registers, the loops with the test in every step are the faster ones (measured: 55 against 67 us
// for the down projection at 256 rows)
constexpr bool mid_whole_turns(int MT) { return MT <= 12; }
constexpr int mid_lds_bytes(int MT) { return mid_xbufs(MT) * 16 * MT * MID_XROW + 16 * MT * (int)sizeof(float); }

// Producer wave P copies the rows 64 P .. of X, macro-step by macro-step, into the ring in LDS.
// chunk c = 64 i + lane of a macro-step: row 64 P + c / 16, 16 bytes at k = 8 (c % 16).  The loads
// go through a buffer resource that ends with the slice's last k of row M - 1 and stand under no
// branch (a branch around a load makes the compiler wait for every load in flight): a row from M
// on has an offset beyond the end and reads zeros, a macro-step beyond the slice reads what lies
// there or zeros and is not used.  The whole offset is the lane's (the hardware checks the
// lane's offset against the end, not the scalar one).
template <int MT, int P>
__device__ __forceinline__ void mid_produce(char *xs, const bf16_t *__restrict__ X, int ldx, int M, int s_begin, int nst, int lane) {
    constexpr int ROWS16 = MT - 4 * P < 4 ? MT - 4 * P : 4;              // tiles of 16 rows that this producer copies
    constexpr int LOADS = ROWS16 * 4;                                     // four rows a load
    constexpr int BUF = 16 * MT * MID_XROW;
    constexpr int XB = mid_xbufs(MT), AHEAD = XB - 1;                     // the copy runs this many macro-steps ahead
    constexpr int D = LOADS <= 8 ? 2 * LCU_MID_XDEPTH : LCU_MID_XDEPTH;   // macro-steps whose loads are on their way (in registers)
    const __amdgpu_buffer_rsrc_t xb = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t *>(X + (size_t)128 * s_begin), 0, (uint32_t)(((size_t)(M - 1) * ldx + 128 * nst) * 2), 0x00020000);
    uint32_t src[LOADS];
    int dst[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int c = 64 * i + lane, tok = 64 * P + (c >> 4), kc = c & 15;
        src[i] = tok < M ? (uint32_t)(tok * ldx + 8 * kc) * 2 : 0x80000000u;
        dst[i] = tok * MID_XROW + 16 * kc;
    }
    u32x4 xr[D][LOADS];
#define MID_LOAD_X(b, step)                                                                                         \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) xr[b][i] =                                                   \
        __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xb, src[i] + (uint32_t)(step) * 256u, 0, 0))
    // the first AHEAD macro-steps go straight into their buffers
#pragma unroll
    for (int b = 0; b < AHEAD; ++b) MID_LOAD_X(b, b);
#pragma unroll
    for (int b = 0; b < AHEAD; ++b)
#pragma unroll
        for (int i = 0; i < LOADS; ++i) *(u32x4 *)(xs + b * BUF + dst[i]) = xr[b][i];
#pragma unroll
    for (int b = 0; b < D; ++b) MID_LOAD_X(b, AHEAD + b);
    lds_barrier();
    // in iteration s: macro-step s + AHEAD goes into buffer (s + AHEAD) % XB, the loads of s + AHEAD + D start.
    // Whole turns of the registers' ring stand under no test of the step (see the consumers' loop)
    int buf = AHEAD;
#define MID_COPY_X(b, cur)                                                                                          \
    do {                                                                                                            \
        _Pragma("unroll") for (int i = 0; i < LOADS; ++i) *(u32x4 *)(xs + buf * BUF + dst[i]) = xr[b][i];          \
        MID_LOAD_X(b, (cur) + AHEAD + D);                                                                           \
        buf = buf == XB - 1 ? 0 : buf + 1;                                                                          \
        lds_barrier();                                                                                              \
    } while (0)
    int s = 0;
    if constexpr (mid_whole_turns(MT)) {
        for (; s + D <= nst; s += D) {
#pragma unroll
            for (int b = 0; b < D; ++b) MID_COPY_X(b, s + b);
        }
    }
    for (; s < nst; s += D) {                      // what is left of the steps (at most one turn after whole ones)
#pragma unroll
        for (int b = 0; b < D; ++b) {
            if (s + b < nst) MID_COPY_X(b, s + b);
        }
    }
#undef MID_COPY_X
#undef MID_LOAD_X
}

template <int NT, int MT, int EPI, bool PACKED, int C>
__global__ void __launch_bounds__((C + mid_producers(MT)) * WAVE)
gemm_mid_kernel(const bf16_t *__restrict__ X, int ldx, const bf16_t *__restrict__ W, int ldw, void *__restrict__ Y, int ldy,
                int M, int N, int K, int steps_per_slice, const float *__restrict__ sumsq_in, int n_in, int norm_width,
                float eps) {
    extern __shared__ __attribute__((aligned(16))) char xs[];      // the ring of X, then the rows' factors
    constexpr int BUF = 16 * MT * MID_XROW;
    constexpr int XB = mid_xbufs(MT);
    float *row_scale = (float *)(xs + XB * BUF);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int l16 = lane & 15, grp = lane >> 4;
    const int steps_total = K / 128;
    const int s_begin = blockIdx.y * steps_per_slice;
    const int s_end = min(steps_total, s_begin + steps_per_slice);
    const int nst = s_end - s_begin;                 // the same for every wave of the workgroup (at least 1)

    if (wave == C) {
        mid_produce<MT, 0>(xs, X, ldx, M, s_begin, nst, lane);
        return;
    }
    if constexpr (MT > 4) {
        if (wave == C + 1) {
            mid_produce<MT, 1>(xs, X, ldx, M, s_begin, nst, lane);
            return;
        }
    }
    if constexpr (MT > 8) {
        if (wave == C + 2) {
            mid_produce<MT, 2>(xs, X, ldx, M, s_begin, nst, lane);
            return;
        }
    }
    if constexpr (MT > 12) {
        if (wave == C + 3) {
            mid_produce<MT, 3>(xs, X, ldx, M, s_begin, nst, lane);
            return;
        }
    }

    // -------------------------------------------------------------------- consumers of W
    // tile t of the wave: rows of W.  SwiGLU: tile 0 a gate tile, tile 1 the up tile N/2 further.
    // the workgroups share the tiles evenly, up to C each: workgroup b takes tiles b n / G .. (b + 1) n / G - 1 of n
    const int n_tiles = (EPI == MID_EPI_SWIGLU ? N / 2 : N) / 16;
    const int tile_begin = (int)((long long)blockIdx.x * n_tiles / gridDim.x);
    const int tile_end = (int)((long long)(blockIdx.x + 1) * n_tiles / gridDim.x);
    const int tile0 = tile_begin + wave;
    const bool live = tile0 < tile_end;              // a wave without a tile reads nothing (a buffer of no bytes) and stores nothing
    // W comes through buffer resources, one per tile, that end with the slice: the loads of the
    // ring stand under no branch, and a macro-step beyond the slice reads zeros (packed) or
    // what lies further in the rows (plain; past the matrix's last row zeros) and is not used.
    __amdgpu_buffer_rsrc_t wb[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int tile = (live ? tile0 : n_tiles - 1) + t * n_tiles;
        wb[t] = PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(W + ((size_t)tile * steps_total + s_begin) * 2048), 0,
                                                             live ? (uint32_t)nst * 4096u : 0u, 0x00020000)
                         : __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(W + (size_t)16 * tile * ldw + (size_t)128 * s_begin), 0,
                                                             live ? (uint32_t)(((size_t)15 * ldw + 128 * nst) * 2) : 0u, 0x00020000);
    }
    // the step and the load within it are constants of the instruction, the lane adds its place once a step
    const uint32_t w_lane = PACKED ? (uint32_t)lane * 16u : (uint32_t)(l16 * ldw + 32 * grp) * 2u;
    constexpr uint32_t w_step = PACKED ? 4096u : 256u, w_j = PACKED ? 1024u : 16u;
    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = f32x4{0.f, 0.f, 0.f, 0.f};
    // the rows' factors: lane group g adds the g-th quarter of a row's shares (sixteen 16-byte loads
    // at a time), the quarters are added in the order of the shuffles
    float scale_ss = 0.f;
    const bool scales = sumsq_in != nullptr && wave < MT;
    if (scales) {
        const int tok = 16 * wave + l16;
        const float *p = sumsq_in + (size_t)(tok < M ? tok : 0) * n_in;
        if ((n_in & 15) == 0) {
            const int q4 = n_in / 16;                         // float4s in a quarter
            const f32x4 *p4 = (const f32x4 *)p + grp * q4;
            for (int i = 0; i < q4; i += 16) {
                f32x4 v[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) v[e] = p4[i + e < q4 ? i + e : q4 - 1];
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (i + e < q4) scale_ss += (v[e][0] + v[e][1]) + (v[e][2] + v[e][3]);
            }
        } else {
            for (int i = grp; i < n_in; i += 4) scale_ss += p[i];
        }
    }
    // loads of W in flight: fewer where the sums take more registers (beyond 128 rows half as many)
    // (measured per shape of the wave's work: with two tiles a wave three stages at 96 rows, four at 128: 54.6 against 58.5 us)
    constexpr int MID_STAGES = MT == 8 && NT == 2 ? MID_STAGE_TILES / 2
                               : (MT > 8 ? MID_STAGE_TILES / 2 : MT > 4 && NT > 1 ? MID_STAGE_TILES * 3 / 4 : MID_STAGE_TILES) / NT;
    constexpr int MCHUNK = MT > 8 ? MT / 2 : MT;          // row tiles whose operands are read from LDS at a time
    u32x4 w[MID_STAGES][NT][4];
#define MID_LOAD_W(i, step)                                                                                     \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) _Pragma("unroll") for (int j = 0; j < 4; ++j) w[i][t][j] =  \
        __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wb[t], w_lane + (uint32_t)(step) * w_step + w_j * j, 0, PACKED ? MID_STREAM : 0))
#pragma unroll
    for (int i = 0; i < MID_STAGES; ++i) MID_LOAD_W(i, i);
    if (scales) {
        scale_ss += __shfl_xor(scale_ss, 16, WAVE);
        scale_ss += __shfl_xor(scale_ss, 32, WAVE);
        if (grp == 0) row_scale[16 * wave + l16] = rsqrtf(scale_ss / (float)norm_width + eps);
    }
    const int x_off = l16 * MID_XROW + 64 * grp;     // the lane's operand of row tile 0, instruction 0
    lds_barrier();                                   // macro-steps 0 and 1 of X are in LDS
    int buf = 0;
#define MID_STEP(i, cur)                                                                                            \
    do {                                                                                                            \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                            \
            _Pragma("unroll") for (int m0 = 0; m0 < MT; m0 += MCHUNK) {                                            \
                u32x4 xf[MCHUNK];                                                                                   \
                _Pragma("unroll") for (int m = 0; m < MCHUNK; ++m)                                                 \
                    xf[m] = *(const u32x4 *)(xs + buf * BUF + x_off + 16 * (m0 + m) * MID_XROW + 16 * j);          \
                _Pragma("unroll") for (int t = 0; t < NT; ++t)                                                     \
                    _Pragma("unroll") for (int m = 0; m < MCHUNK; ++m)                                             \
                        acc[t][m0 + m] = mid_mfma(w[i][t][j], xf[m], acc[t][m0 + m]);                               \
            }                                                                                                       \
        }                                                                                                           \
        MID_LOAD_W(i, (cur) + MID_STAGES);                                                                          \
        buf = buf == XB - 1 ? 0 : buf + 1;                                                                          \
        lds_barrier();                                                                                              \
    } while (0)
    // Whole turns of the ring stand under no test of the step: the compiler then counts the loads that a turn has
    // issued when it waits for the oldest one.  With a test around every step it assumed that none of them had been
    // issued and waited for ever more of the ring, until at a turn's last step nothing was in flight.
    int s = 0;
    if constexpr (mid_whole_turns(MT)) {
        for (; s + MID_STAGES <= nst; s += MID_STAGES) {
#pragma unroll
            for (int i = 0; i < MID_STAGES; ++i) MID_STEP(i, s + i);
        }
    }
    for (; s < nst; s += MID_STAGES) {             // what is left of the steps (at most one turn after whole ones)
#pragma unroll
        for (int i = 0; i < MID_STAGES; ++i) {
            if (s + i < nst) MID_STEP(i, s + i);
        }
    }
#undef MID_STEP
#undef MID_LOAD_W
    if (!live) return;
    // ---- epilogue: the lane holds, per tile, features 4 grp + r of token 16 m + l16
    if (sumsq_in != nullptr) {                       // (the factors were written before the loop's barriers)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float rs = row_scale[16 * m + l16];
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][m][r] *= rs;
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int tok = 16 * m + l16;
        if (tok >= M) continue;
        const int n = 16 * tile0 + 4 * grp;
        if (EPI == MID_EPI_SWIGLU) {
            float o[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float gate = acc[0][m][r], up = acc[NT - 1][m][r];
                o[r] = gate * (1.0f / (1.0f + expf(-gate))) * up;
            }
            uint2 pk = {pack2_bf16(o[0], o[1]), pack2_bf16(o[2], o[3])};
            *(uint2 *)((bf16_t *)Y + (size_t)tok * ldy + n) = pk;
        } else if (EPI == MID_EPI_BF16) {
            uint2 pk = {pack2_bf16(acc[0][m][0], acc[0][m][1]), pack2_bf16(acc[0][m][2], acc[0][m][3])};
            *(uint2 *)((bf16_t *)Y + (size_t)tok * ldy + n) = pk;
        } else {
            float *plane = (float *)Y + (size_t)blockIdx.y * M * ldy;
            *(f32x4 *)(plane + (size_t)tok * ldy + n) = acc[0][m];
        }
    }
}

// The number of compute units of the current device (asked once per device).
static int mid_compute_units() {
    static int units[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (units[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
        units[dev] = n > 0 ? n : -1;
    }
    return units[dev] > 0 ? units[dev] : 0;
}

struct MidScale {
    const float *sumsq_in;
    int n_in, norm_width;
    float eps;
};

// The number of consumer waves: four; two for SwiGLU with up to 32 rows (workgroups of two tiles, two to a compute
// unit: 39.8 against 44.0 us at 24 rows of a 28,672-row gate/up matrix).
template <int NT, int EPI, int C>
static int mid_launch_c(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K, int packed,
                        int slices, const MidScale &sc, hipStream_t stream) {
    const int n_tiles = (EPI == MID_EPI_SWIGLU ? N / 2 : N) / 16;
    const int steps = K / 128, per = (steps + slices - 1) / slices;
    // workgroups: as many as take C tiles each; where K is not cut and a workgroup reads few rows (up to 64), the next
    // multiple of the number of compute units, so that none of them idles (28,672 rows of gate/up are 224 workgroups of
    // four tiles: as 256 workgroups of three and four tiles 41.8 against 45.2 us at 64 rows; beyond 64 rows more
    // workgroups cost more in reads of X than they gain)
    int groups = (n_tiles + C - 1) / C;
    if (slices == 1 && M <= 64) {
        const int units = mid_compute_units();
        if (units > 0) groups = min(n_tiles, (groups + units - 1) / units * units);
    }
    const dim3 grid(groups, (steps + per - 1) / per);
    // the ring of 65 to 256 rows takes more LDS than a kernel has without asking
#define GO(MT_, P_)                                                                                                         \
    do {                                                                                                                    \
        auto kernel = gemm_mid_kernel<NT, MT_, EPI, P_, C>;                                                                 \
        if (mid_lds_bytes(MT_) > 64 * 1024) {                                                                               \
            static bool asked = false;                                                                                      \
            if (!asked) {                                                                                                   \
                hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,      \
                                                   mid_lds_bytes(MT_));                                                     \
                if (e != hipSuccess) return (int)e;                                                                         \
                asked = true;                                                                                               \
            }                                                                                                               \
        }                                                                                                                   \
        kernel<<<grid, dim3((C + mid_producers(MT_)) * WAVE), mid_lds_bytes(MT_), stream>>>(                                \
            (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, per, sc.sumsq_in, sc.n_in, sc.norm_width, sc.eps); \
    } while (0)
#define GO_MT(MT_)                 \
    do {                           \
        if (packed) GO(MT_, true); \
        else GO(MT_, false);       \
    } while (0)
    if constexpr (C < MID_CONSUMERS) {
        GO_MT(2);                                   // (chosen for up to 32 rows only)
    } else {
        if (M <= 32) GO_MT(2);
        else if (M <= 48) GO_MT(3);
        else if (M <= 64) GO_MT(4);
        else if (M <= 96) GO_MT(6);
        else if (M <= 128) GO_MT(8);
        else if (M <= 192) GO_MT(12);
        else GO_MT(16);
    }
#undef GO_MT
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

template <int NT, int EPI>
static int mid_launch(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K, int packed,
                      int slices, const MidScale &sc, hipStream_t stream) {
    if constexpr (EPI == MID_EPI_SWIGLU && MID_CONSUMERS == 4) {
        if (M <= 32) return mid_launch_c<NT, EPI, 2>(X, ldx, W, ldw, Y, ldy, M, N, K, packed, slices, sc, stream);
    }
    return mid_launch_c<NT, EPI, MID_CONSUMERS>(X, ldx, W, ldw, Y, ldy, M, N, K, packed, slices, sc, stream);
}

// X: [M, K] bfloat16 rows ldx apart, M <= 256 (rows that wait for their normalisation: M <= 64); W: [N, K] bfloat16, rows ldw apart or packed; K a
// multiple of 128, N of 16 (SwiGLU: of 32; W holds N/2 gate rows, then N/2 up rows).
// epilogue MID_EPI_BF16: Y [M, N] bfloat16 rows ldy apart (slices must be 1);
//          MID_EPI_SWIGLU: Y [M, N/2] bfloat16 = silu(gate) * up (slices must be 1);
//          MID_EPI_PARTIAL_F32: Y [slices_used][M][ldy] float32, plane s the sum over slice s of K;
//          the planes that exist are ceil(steps / ceil(steps / slices)) with steps = K / 128
//          (lcu_gemm_mid_planes gives the number).
LCU_API int lcu_gemm_mid_planes(int K, int slices) {
    if (K <= 0 || K % 128 || slices <= 0) return LCU_BAD_ARGUMENT;
    const int steps = K / 128, per = (steps + slices - 1) / slices;
    return (steps + per - 1) / per;
}

static int mid_bf16(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K, int epilogue,
                    int slices, int w_packed, const MidScale &sc, hipStream_t stream) {
    if (M <= 0 || N <= 0) return LCU_OK;
    if (M > 256 || (sc.sumsq_in && M > 64) || K <= 0 || K % 128 || N % 16 || ldx % 8 || ldx < K || slices <= 0 || slices > 64) return LCU_BAD_ARGUMENT;
    if (!w_packed && (ldw % 8 || ldw < K)) return LCU_BAD_ARGUMENT;
    if ((uintptr_t)X % 16 || (uintptr_t)W % 16 || (uintptr_t)Y % 16 || (uintptr_t)sc.sumsq_in % 16) return LCU_BAD_ARGUMENT;
    switch (epilogue) {
    case MID_EPI_BF16:
        if (slices != 1 || ldy < N || ldy % 4) return LCU_BAD_ARGUMENT;
        return mid_launch<1, MID_EPI_BF16>(X, ldx, W, ldw, Y, ldy, M, N, K, w_packed, 1, sc, stream);
    case MID_EPI_PARTIAL_F32:
        if (ldy < N || ldy % 4) return LCU_BAD_ARGUMENT;
        return mid_launch<1, MID_EPI_PARTIAL_F32>(X, ldx, W, ldw, Y, ldy, M, N, K, w_packed, slices, sc, stream);
    case MID_EPI_SWIGLU:
        if (slices != 1 || N % 32 || ldy < N / 2 || ldy % 4) return LCU_BAD_ARGUMENT;
        return mid_launch<2, MID_EPI_SWIGLU>(X, ldx, W, ldw, Y, ldy, M, N, K, w_packed, 1, sc, stream);
    default: return LCU_BAD_ARGUMENT;
    }
}

LCU_API int lcu_gemm_mid_bf16(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K,
                              int epilogue, int slices, int w_packed, hipStream_t stream) {
    const MidScale none = {nullptr, 0, 0, 0.f};
    return mid_bf16(X, ldx, W, ldw, Y, ldy, M, N, K, epilogue, slices, w_packed, none, stream);
}

// The same with rows of X that wait for their normalisation: row i of the product is multiplied by
// rsqrt(sum(sumsq_in[i][0 .. n_in)) / norm_width + eps) before the epilogue.  sumsq_in: [M][n_in] float32.
LCU_API int lcu_gemm_mid_bf16_scaled(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K,
                                     int epilogue, int slices, int w_packed, const float *sumsq_in, int n_in,
                                     int norm_width, float eps, hipStream_t stream) {
    if (!sumsq_in || n_in <= 0 || norm_width <= 0) return LCU_BAD_ARGUMENT;
    const MidScale sc = {sumsq_in, n_in, norm_width, eps};
    return mid_bf16(X, ldx, W, ldw, Y, ldy, M, N, K, epilogue, slices, w_packed, sc, stream);
}

#if LCU_MID_CONSUMERS == 4
// ------------------------------------------------------------------------------------------------
// The q, k, v product of an attention layer with the rotation and the cache write in its epilogue,
// for more rows than gemm_skinny.hip's takes.  W holds the rows of the q heads, the k heads and the v
// heads, head_dim each.  A rotation pairs dim i of a head with dim i + head_dim/2, so a workgroup takes
// two tiles of one head, dims 16 c .. and head_dim/2 + 16 c .., over all of K; with so few features a
// workgroup there are workgroups enough (192 for 48 heads of 128) without cutting K over workgroups,
// which a rotation in the epilogue could not have.  Instead the four consumer waves share each
// macro-step of 128 k: wave w multiplies the k that the w-th matrix instruction of a macro-step takes
// (in the packed layout the w-th KB of a tile's 4 KB block), all four read the same rows of X from the
// ring, and at the end they add their sums through LDS in the order of the waves.  Wave w then holds
// the row tiles w, w + 4, .. of both tiles: it rounds q and k to bfloat16 (as the plain product
// stores them for the rotation kernel), rotates them by the token's position, writes q to q_out and
// k and v into the token's place in its page.
template <int MT, bool PACKED>
__global__ void __launch_bounds__((MID_CONSUMERS + mid_producers(MT)) * WAVE)
gemm_mid_qkv_kernel(const bf16_t *__restrict__ X, int ldx, const bf16_t *__restrict__ W, int ldw, int M, int K,
                    bf16_t *__restrict__ q_out, int ldq, const int *__restrict__ positions, const int *__restrict__ slots,
                    const float *__restrict__ cos_t, const float *__restrict__ sin_t, int max_pos, bf16_t *__restrict__ cache,
                    int heads, int kv_heads, int head_dim, int page) {
    static_assert(MID_CONSUMERS == 4, "the four matrix instructions of a macro-step go to four waves");
    extern __shared__ __attribute__((aligned(16))) char xs[];      // the ring of X; at the end the waves' sums
    constexpr int BUF = 16 * MT * MID_XROW;
    constexpr int XB = mid_xbufs(MT);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int l16 = lane & 15, grp = lane >> 4;
    const int nst = K / 128;
    if (wave == MID_CONSUMERS) {
        mid_produce<MT, 0>(xs, X, ldx, M, 0, nst, lane);
        return;
    }
    if constexpr (MT > 4) {
        if (wave == MID_CONSUMERS + 1) {
            mid_produce<MT, 1>(xs, X, ldx, M, 0, nst, lane);
            return;
        }
    }
    if constexpr (MT > 8) {
        if (wave == MID_CONSUMERS + 2) {
            mid_produce<MT, 2>(xs, X, ldx, M, 0, nst, lane);
            return;
        }
    }
    if constexpr (MT > 12) {
        if (wave == MID_CONSUMERS + 3) {
            mid_produce<MT, 3>(xs, X, ldx, M, 0, nst, lane);
            return;
        }
    }
    const int per_head = head_dim / 32;
    const int head = blockIdx.x / per_head, c = blockIdx.x % per_head;
    __amdgpu_buffer_rsrc_t wb[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int tile = head * (head_dim / 16) + c + t * per_head;
        wb[t] = PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(W + (size_t)tile * nst * 2048), 0, (uint32_t)nst * 4096u, 0x00020000)
                       : __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(W + (size_t)16 * tile * ldw), 0,
                                                           (uint32_t)(((size_t)15 * ldw + 128 * nst) * 2), 0x00020000);
    }
    const uint32_t w_lane = PACKED ? (uint32_t)lane * 16u + 1024u * wave : (uint32_t)(l16 * ldw + 32 * grp) * 2u + 16u * wave;
    constexpr uint32_t w_step = PACKED ? 4096u : 256u;
    f32x4 acc[2][MT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int STAGES = MT > 8 ? 8 : 16;            // macro-steps whose loads of W (1 KB a tile) are in flight
    constexpr int MCHUNK = MT > 8 ? MT / 2 : MT;       // row tiles whose operands are read from LDS at a time
    u32x4 w[STAGES][2];
#define QKV_LOAD_W(i, step)                                                                             \
    _Pragma("unroll") for (int t = 0; t < 2; ++t) w[i][t] = __builtin_bit_cast(                        \
        u32x4, __builtin_amdgcn_raw_buffer_load_b128(wb[t], w_lane + (uint32_t)(step) * w_step, 0, PACKED ? MID_STREAM : 0))
#pragma unroll
    for (int i = 0; i < STAGES; ++i) QKV_LOAD_W(i, i);
    const int x_off = l16 * MID_XROW + 64 * grp + 16 * wave;
    lds_barrier();
    int buf = 0;
#define QKV_STEP(i, cur)                                                                                      \
    do {                                                                                                      \
        _Pragma("unroll") for (int m0 = 0; m0 < MT; m0 += MCHUNK) {                                          \
            u32x4 xf[MCHUNK];                                                                                 \
            _Pragma("unroll") for (int m = 0; m < MCHUNK; ++m)                                               \
                xf[m] = *(const u32x4 *)(xs + buf * BUF + x_off + 16 * (m0 + m) * MID_XROW);                 \
            _Pragma("unroll") for (int t = 0; t < 2; ++t)                                                    \
                _Pragma("unroll") for (int m = 0; m < MCHUNK; ++m) acc[t][m0 + m] = mid_mfma(w[i][t], xf[m], acc[t][m0 + m]); \
        }                                                                                                     \
        QKV_LOAD_W(i, (cur) + STAGES);                                                                        \
        buf = buf == XB - 1 ? 0 : buf + 1;                                                                    \
        lds_barrier();                                                                                        \
    } while (0)
    // whole turns of the ring stand under no branch: the compiler then counts the loads of a turn that are on their
    // way when it waits for the oldest (with a test of the step around each, it assumed none of them and let the
    // ring run empty once a turn)
    int s = 0;
    if constexpr (mid_whole_turns(MT)) {
        for (; s + STAGES <= nst; s += STAGES) {
#pragma unroll
            for (int i = 0; i < STAGES; ++i) QKV_STEP(i, s + i);
        }
    }
    for (; s < nst; s += STAGES) {                 // what is left of the steps (at most one turn after whole ones)
#pragma unroll
        for (int i = 0; i < STAGES; ++i) {
            if (s + i < nst) QKV_STEP(i, s + i);
        }
    }
#undef QKV_STEP
#undef QKV_LOAD_W
    // every wave has passed the last barrier: nobody reads the ring any more, the producers have ended.
    // The waves' sums: [wave][tile][row tile][lane], 16 bytes each
    f32x4 *sums = (f32x4 *)xs;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) sums[((wave * 2 + t) * MT + m) * WAVE + lane] = acc[t][m];
    lds_barrier();
    const int half_dim = head_dim / 2;
    const bool is_q = head < heads, is_k = !is_q && head < heads + kv_heads;
#pragma unroll
    for (int mi = 0; mi < (MT + MID_CONSUMERS - 1) / MID_CONSUMERS; ++mi) {
        const int m = wave + MID_CONSUMERS * mi;
        if (m >= MT) break;
        f32x4 sum[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            sum[t] = sums[((0 * 2 + t) * MT + m) * WAVE + lane];
#pragma unroll
            for (int v = 1; v < MID_CONSUMERS; ++v) {
                const f32x4 o = sums[((v * 2 + t) * MT + m) * WAVE + lane];
                sum[t][0] += o[0]; sum[t][1] += o[1]; sum[t][2] += o[2]; sum[t][3] += o[3];
            }
        }
        // the lane holds dims i0 .. i0 + 3 (tile 0) and head_dim/2 + i0 .. (tile 1) of token 16 m + l16
        const int tok = 16 * m + l16;
        if (tok >= M) continue;
        const int i0 = 16 * c + 4 * grp;
        const int pos = positions[tok];
        const bool in_table = pos >= 0 && pos < max_pos;
        const int slot = slots ? slots[tok] : -1;
        bf16_t *pg = nullptr;
        int place = 0;
        if (!is_q && slot >= 0) {
            pg = cache + (size_t)(slot / page) * kv_page_elems(kv_heads, head_dim, page);
            place = slot % page;
        }
        bf16_t va[4], vb[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            // rounded to bfloat16 before the rotation, as the plain product stores them for the rotation
            // kernel: a token's query and key are made the same way whichever kernel makes them
            float a = to_f32(from_f32<bf16_t>(sum[0][r])), b = to_f32(from_f32<bf16_t>(sum[1][r]));
            if (is_q || is_k) {
                float cs = __uint_as_float(0x7fc00000u), sn = cs;         // a position outside the table gives NaN
                if (in_table) { cs = cos_t[(size_t)pos * half_dim + i0 + r]; sn = sin_t[(size_t)pos * half_dim + i0 + r]; }
                float ra, rb;
                rotate_pair(a, b, cs, sn, ra, rb);
                a = ra; b = rb;
            }
            va[r] = from_f32<bf16_t>(a);
            vb[r] = from_f32<bf16_t>(b);
        }
        if (is_q) {
            bf16_t *qo = q_out + (size_t)tok * ldq + (size_t)head * head_dim;
#pragma unroll
            for (int r = 0; r < 4; ++r) { qo[i0 + r] = va[r]; qo[i0 + half_dim + r] = vb[r]; }
        } else if (pg) {
            if (is_k) {
                const int kvh = head - heads;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pg[kv_key_offset(kvh, place, i0 + r, head_dim, page)] = va[r];
                    pg[kv_key_offset(kvh, place, i0 + half_dim + r, head_dim, page)] = vb[r];
                }
            } else {
                const int kvh = head - heads - kv_heads;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pg[kv_value_offset(kv_heads, kvh, place, i0 + r, head_dim, page)] = va[r];
                    pg[kv_value_offset(kv_heads, kvh, place, i0 + half_dim + r, head_dim, page)] = vb[r];
                }
            }
        }
    }
}

#endif

// X: [M, K] bfloat16 rows ldx apart, M <= 256, K a multiple of 128; W: [(heads + 2 kv_heads) * head_dim, K] bfloat16 (q heads,
// then k heads, then v heads), rows ldw apart or packed; head_dim a multiple of 32.  q_out: [M, heads * head_dim] rows
// ldq apart takes the rotated queries; the rotated keys and the values go to cache (this layer's pages, laid out as
// kv_layout.h says) at slots[m] (page * page_size + place; negative or slots null: nothing is stored).  cos_t, sin_t:
// [max_pos, head_dim / 2] float32; pairs are (i, i + head_dim / 2).
LCU_API int lcu_gemm_mid_bf16_qkv_rope(const void *X, int ldx, const void *W, int ldw, int M, int K, void *q_out, int ldq,
                                       const int *positions, const int *slots, const float *cos_t, const float *sin_t,
                                       int max_pos, void *cache, int heads, int kv_heads, int head_dim, int page,
                                       int w_packed, hipStream_t stream) {
    if (M <= 0) return LCU_OK;
    if (M > 256 || K <= 0 || K % 128 || heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim % 32 || page <= 0 || page % 8 ||
        !q_out || !positions || !cos_t || !sin_t || max_pos <= 0 || !cache || ldq < heads * head_dim || ldx % 8 || ldx < K)
        return LCU_BAD_ARGUMENT;
    if (!w_packed && (ldw % 8 || ldw < K)) return LCU_BAD_ARGUMENT;
    if ((uintptr_t)X % 16 || (uintptr_t)W % 16) return LCU_BAD_ARGUMENT;
#if LCU_MID_CONSUMERS == 4
    const dim3 grid((heads + 2 * kv_heads) * (head_dim / 32));
#define GO(MT_, P_)                                                                                                         \
    do {                                                                                                                    \
        auto kernel = gemm_mid_qkv_kernel<MT_, P_>;                                                                         \
        constexpr int lds = mid_xbufs(MT_) * 16 * MT_ * MID_XROW;                                                           \
        static_assert(lds >= MID_CONSUMERS * 2 * MT_ * WAVE * 16, "the waves' sums lie over the ring");                     \
        if (lds > 64 * 1024) {                                                                                              \
            static bool asked = false;                                                                                      \
            if (!asked) {                                                                                                   \
                hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds); \
                if (e != hipSuccess) return (int)e;                                                                         \
                asked = true;                                                                                               \
            }                                                                                                               \
        }                                                                                                                   \
        kernel<<<grid, dim3((MID_CONSUMERS + mid_producers(MT_)) * WAVE), lds, stream>>>(                                   \
            (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, M, K, (bf16_t *)q_out, ldq, positions, slots, cos_t, sin_t,    \
            max_pos, (bf16_t *)cache, heads, kv_heads, head_dim, page);                                                     \
    } while (0)
#define GO_MT(MT_)                   \
    do {                             \
        if (w_packed) GO(MT_, true); \
        else GO(MT_, false);         \
    } while (0)
    if (M <= 32) GO_MT(2);
    else if (M <= 48) GO_MT(3);
    else if (M <= 64) GO_MT(4);
    else if (M <= 96) GO_MT(6);
    else if (M <= 128) GO_MT(8);
    else if (M <= 192) GO_MT(12);
    else GO_MT(16);
#undef GO_MT
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
#else
    return LCU_BAD_ARGUMENT;       // an experimental build with another number of consumer waves has no such kernel
#endif
}

#if LCU_MID_CONSUMERS == 4
// ------------------------------------------------------------------------------------------------
// The product that ends a branch, with the residual sum and the next norm's weight in its epilogue, as
// gemm_skinny.hip has it for few rows: residual[M, N] += X W^T (32-bit, in place), h = bfloat16(residual * norm_w),
// not yet normalised, and sumsq[M][N / 16], each workgroup's share of the rows' sums of squares (whoever multiplies h
// next applies rsqrt(sum of a row's shares / N + eps) in its epilogue).  A sum of squares over a row needs the whole
// of K under it, so K is not cut over workgroups: a workgroup takes one tile of 16 output features over all of K, and
// its four consumer waves share each macro-step as in the q, k, v kernel above.  For products with a short K (the
// output projection): every workgroup reads all rows of X.
template <int MT, bool PACKED>
__global__ void __launch_bounds__((MID_CONSUMERS + mid_producers(MT)) * WAVE)
gemm_mid_add_norm_kernel(const bf16_t *__restrict__ X, int ldx, const bf16_t *__restrict__ W, int ldw, float *__restrict__ residual,
                         int ldr, int M, int N, int K, const void *__restrict__ norm_w, int norm_w_type, bf16_t *__restrict__ h_out,
                         int ldh, float *__restrict__ sumsq_out) {
    extern __shared__ __attribute__((aligned(16))) char xs[];      // the ring of X; at the end the waves' sums
    constexpr int BUF = 16 * MT * MID_XROW;
    constexpr int XB = mid_xbufs(MT);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int l16 = lane & 15, grp = lane >> 4;
    const int nst = K / 128;
    if (wave == MID_CONSUMERS) {
        mid_produce<MT, 0>(xs, X, ldx, M, 0, nst, lane);
        return;
    }
    const int tile = blockIdx.x;
    const __amdgpu_buffer_rsrc_t wb =
        PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(W + (size_t)tile * nst * 2048), 0, (uint32_t)nst * 4096u, 0x00020000)
               : __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(W + (size_t)16 * tile * ldw), 0,
                                                   (uint32_t)(((size_t)15 * ldw + 128 * nst) * 2), 0x00020000);
    const uint32_t w_lane = PACKED ? (uint32_t)lane * 16u + 1024u * wave : (uint32_t)(l16 * ldw + 32 * grp) * 2u + 16u * wave;
    constexpr uint32_t w_step = PACKED ? 4096u : 256u;
    f32x4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int STAGES = 16;                         // macro-steps whose loads of W (1 KB) are in flight
    u32x4 w[STAGES];
#define AN_LOAD_W(i, step) \
    w[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wb, w_lane + (uint32_t)(step) * w_step, 0, PACKED ? MID_STREAM : 0))
#pragma unroll
    for (int i = 0; i < STAGES; ++i) AN_LOAD_W(i, i);
    const int x_off = l16 * MID_XROW + 64 * grp + 16 * wave;
    lds_barrier();
    int buf = 0;
#define AN_STEP(i, cur)                                                                                       \
    do {                                                                                                      \
        u32x4 xf[MT];                                                                                         \
        _Pragma("unroll") for (int m = 0; m < MT; ++m) xf[m] = *(const u32x4 *)(xs + buf * BUF + x_off + 16 * m * MID_XROW); \
        _Pragma("unroll") for (int m = 0; m < MT; ++m) acc[m] = mid_mfma(w[i], xf[m], acc[m]);                \
        AN_LOAD_W(i, (cur) + STAGES);                                                                         \
        buf = buf == XB - 1 ? 0 : buf + 1;                                                                    \
        lds_barrier();                                                                                        \
    } while (0)
    int s = 0;
    for (; s + STAGES <= nst; s += STAGES) {           // whole turns of the ring under no test of the step (see above)
#pragma unroll
        for (int i = 0; i < STAGES; ++i) AN_STEP(i, s + i);
    }
    for (; s < nst; s += STAGES) {
#pragma unroll
        for (int i = 0; i < STAGES; ++i) {
            if (s + i < nst) AN_STEP(i, s + i);
        }
    }
#undef AN_STEP
#undef AN_LOAD_W
    // the waves' sums: [wave][row tile][lane], 16 bytes each; wave w then holds the row tiles w, w + 4, ..
    f32x4 *sums = (f32x4 *)xs;
#pragma unroll
    for (int m = 0; m < MT; ++m) sums[(wave * MT + m) * WAVE + lane] = acc[m];
    lds_barrier();
    const int parts = gridDim.x;
#pragma unroll
    for (int mi = 0; mi < (MT + MID_CONSUMERS - 1) / MID_CONSUMERS; ++mi) {
        const int m = wave + MID_CONSUMERS * mi;
        if (m >= MT) break;
        f32x4 sum = sums[(0 * MT + m) * WAVE + lane];
#pragma unroll
        for (int v = 1; v < MID_CONSUMERS; ++v) {
            const f32x4 o = sums[(v * MT + m) * WAVE + lane];
            sum[0] += o[0]; sum[1] += o[1]; sum[2] += o[2]; sum[3] += o[3];
        }
        // the lane holds features n0 .. n0 + 3 of token 16 m + l16
        const int tok = 16 * m + l16, n0 = 16 * tile + 4 * grp;
        float ss = 0.f;
        if (tok < M) {
            f32x4 *res = (f32x4 *)(residual + (size_t)tok * ldr + n0);
            f32x4 xn = *res;
            xn[0] += sum[0]; xn[1] += sum[1]; xn[2] += sum[2]; xn[3] += sum[3];
            *res = xn;
            float wn[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                ss += xn[r] * xn[r];
                wn[r] = norm_w_type == LCU_F32 ? ((const float *)norm_w)[n0 + r] : to_f32(((const bf16_t *)norm_w)[n0 + r]);
            }
            uint2 pk = {pack2_bf16(xn[0] * wn[0], xn[1] * wn[1]), pack2_bf16(xn[2] * wn[2], xn[3] * wn[3])};
            *(uint2 *)(h_out + (size_t)tok * ldh + n0) = pk;
        }
        ss += __shfl_xor(ss, 16, WAVE);                // every lane takes part: the others bring zero
        ss += __shfl_xor(ss, 32, WAVE);
        if (grp == 0 && tok < M) sumsq_out[(size_t)tok * parts + blockIdx.x] = ss;
    }
}
#endif

// X: [M, K] bfloat16 rows ldx apart, M <= 64, K a multiple of 128; W: [N, K] bfloat16, N a multiple of 16, rows ldw apart or
// packed.  residual: [M, N] float32 rows ldr apart (a multiple of 4), updated in place; norm_w: [N] float32 or bfloat16
// (norm_w_type LCU_F32 or LCU_BF16); h_out: [M, N] bfloat16 rows ldh apart (a multiple of 4); sumsq_out: [M][N / 16] float32.
LCU_API int lcu_gemm_mid_bf16_add_norm(const void *X, int ldx, const void *W, int ldw, float *residual, int ldr, int M, int N, int K,
                                       const void *norm_w, int norm_w_type, void *h_out, int ldh, float *sumsq_out, int w_packed,
                                       hipStream_t stream) {
    if (M <= 0 || N <= 0) return LCU_OK;
    if (M > 64 || K <= 0 || K % 128 || N % 16 || ldx % 8 || ldx < K || ldr < N || ldr % 4 || ldh < N || ldh % 4 || !residual || !norm_w ||
        !h_out || !sumsq_out || (norm_w_type != LCU_F32 && norm_w_type != LCU_BF16))
        return LCU_BAD_ARGUMENT;
    if (!w_packed && (ldw % 8 || ldw < K)) return LCU_BAD_ARGUMENT;
    if ((uintptr_t)X % 16 || (uintptr_t)W % 16 || (uintptr_t)residual % 16 || (uintptr_t)h_out % 8) return LCU_BAD_ARGUMENT;
#if LCU_MID_CONSUMERS == 4
    const dim3 grid(N / 16);
#define GO(MT_, P_)                                                                                                          \
    do {                                                                                                                     \
        constexpr int lds = mid_xbufs(MT_) * 16 * MT_ * MID_XROW;                                                            \
        static_assert(lds >= MID_CONSUMERS * MT_ * WAVE * 16 && lds <= 64 * 1024, "the waves' sums lie over the ring");      \
        gemm_mid_add_norm_kernel<MT_, P_><<<grid, dim3((MID_CONSUMERS + mid_producers(MT_)) * WAVE), lds, stream>>>(         \
            (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, residual, ldr, M, N, K, norm_w, norm_w_type, (bf16_t *)h_out, ldh, sumsq_out); \
    } while (0)
#define GO_MT(MT_)                   \
    do {                             \
        if (w_packed) GO(MT_, true); \
        else GO(MT_, false);         \
    } while (0)
    if (M <= 16) GO_MT(1);
    else if (M <= 32) GO_MT(2);
    else if (M <= 48) GO_MT(3);
    else GO_MT(4);
#undef GO_MT
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
#else
    return LCU_BAD_ARGUMENT;       // an experimental build with another number of consumer waves has no such kernel
#endif
}
