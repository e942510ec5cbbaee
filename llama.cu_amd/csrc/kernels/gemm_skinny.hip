// Y[M, N] = X[M, K] * W[N, K]^T for few rows (decoding: M <= 32), bfloat16 operands,
// 32-bit accumulation on the matrix cores.  The work is streaming W once from HBM, so
// the kernel is laid out around W's loads:
//
//   * a workgroup of 4 or 8 waves owns NT tiles of 16 output features (rows of W) and walks
//     the whole K: no sum crosses workgroups, results do not depend on the grid, and
//     the epilogue can be fused;
//   * K goes in macro-steps of 128; the waves take macro-steps in turn; in a macro-step
//     lane group g of a wave reads the 64 contiguous bytes k0 + 32g .. k0 + 32g + 31 of
//     its row as four 16-byte loads, one per matrix instruction (which k a slot of the
//     instruction holds is free, as long as W and X agree), so the four waves read 1 KB
//     of a row back to back;
//   * a wave keeps the loads of several macro-steps in flight while it multiplies one;
//   * v_mfma_f32_16x16x32_bf16 with A = W tile, B = X^T: the 16 columns are 16 tokens,
//     MT such tiles for up to 32 tokens (more rows go to gemm_mid.hip, which shares them through LDS).
// The waves' partial sums are added in LDS in a fixed order.
//
// W may also be given packed (lcu_pack_weight / the wrapper's pack_weight): the 16 x 128 block
// of a tile and a macro-step lies in 4 KB of its own, ordered [j][lane][8] as the lanes load it,
// the blocks of a tile one after the other.  Then every load instruction of a wave reads 1 KB
// in one piece and a workgroup streams one contiguous run of memory, which HBM serves
// faster than pieces of 256 bytes out of 16 or 32 rows that lie kilobytes apart.
//
// Epilogues: store bfloat16; store float32 (logits); add into float32 (the residual
// stream); SwiGLU, where the workgroup's two tiles are the gate rows n and the up rows
// n + N/2 of one matrix and silu(gate) * up is stored.
#include "common.h"
#include "kv_layout.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ADD_F32 = 2, EPI_SWIGLU = 3, EPI_ADD_NORM = 4, EPI_QKV_ROPE = 5 };

// What two epilogues need beside Y, so that no kernel stands between a projection that ends
// a branch and the product that follows the next norm:
//   EPI_ADD_NORM: Y is the float32 residual stream and takes the product in; the new rows times
//     the norm's weight go to h_out as bfloat16, *not yet normalised*, and the workgroup's
//     share of each row's sum of squares goes to sumsq_out[row][workgroup].
//   row scale (any other epilogue, sumsq_in not null): the rows of X are such rows; a row of
//     the product is multiplied by rsqrt(sum of its shares / norm_width + eps) before the
//     epilogue (the normalisation is a factor per row, so it commutes with the product).
//   EPI_QKV_ROPE: W holds the q, k and v projections (rows q heads, k heads, v heads, head_dim
//     each).  A workgroup's two tiles are 16 dims of a head and the 16 dims head_dim/2 further,
//     the pairs of the rotation (half-split pairing over the whole head): the epilogue rotates q
//     and k by the token's position, writes q to q_out and k and v straight into the token's
//     place in the paged cache.  No rotation kernel runs after this product.
// The shares are added in a fixed order: no atomics, results do not depend on timing.
struct SkinnyExtra {
    const void *norm_w;        // [N] norm weight of EPI_ADD_NORM
    int norm_w_type;           // LCU_F32 or LCU_BF16
    bf16_t *h_out;             // [M, N] rows ldh apart
    int ldh;
    float *sumsq_out;          // [M][gridDim.x]
    const float *sumsq_in;     // [M][n_in] or null
    int n_in;
    int norm_width;
    float eps;
    // EPI_QKV_ROPE
    const int *positions;      // [M]
    const int *slots;          // [M] page * page_size + place, or -1: store nothing
    const float *cos_t, *sin_t;  // [max_pos, head_dim / 2]
    int max_pos;
    bf16_t *cache;             // this layer's pages
    bf16_t *q_out;             // [M, heads * head_dim] rows ldq apart
    int ldq;
    int heads, kv_heads, head_dim, page;
};

__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <int NT, int MT>
struct Frag {
    u32x4 w[NT][4];
    u32x4 x[MT][4];
};

// A weight is read once per product and never again before the caches have turned over: the loads of a packed
// weight are marked non-temporal, so that they do not displace what is used again (the rows, the next kernel's
// operands).  A kernel that only reads memory moves 6.2 to 6.4 TB/s of a 235 MB stretch with such loads and 5.7
// with ordinary ones.  Only where a load instruction of a wave takes whole 128-byte lines, as it does from a packed
// weight: from plain rows, where eight instructions share a line, such loads fetch the line again and again (the
// decode step of 8 requests took 5.5 ms with them and plain rows).
__device__ __forceinline__ u32x4 stream_load(const u32x4 *p) { return __builtin_nontemporal_load(p); }

// The lane's loads of macro-step s: k = 128 s + 32 grp + 8 j .. + 7 for j = 0..3.
template <int NT, int MT, bool PACKED>
__device__ __forceinline__ void load_frag(Frag<NT, MT> &f, const bf16_t *const (&wrow)[NT], const bf16_t *const (&xrow)[MT],
                                          const bool (&xvalid)[MT], int s, int grp, int K) {
    const int kb = 128 * s + 32 * grp;
    const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
    if (128 * (s + 1) <= K) {
        // packed: wrow is the lane's place in the tile's first block; blocks are 2048 elements,
        // the four loads of a block 512 apart
        const int w0 = PACKED ? 2048 * s : kb, wj = PACKED ? 512 : 8;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                f.w[t][j] = PACKED ? stream_load((const u32x4 *)(wrow[t] + w0 + wj * j)) : *(const u32x4 *)(wrow[t] + w0 + wj * j);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < 4; ++j) f.x[m][j] = xvalid[m] ? *(const u32x4 *)(xrow[m] + kb + 8 * j) : zero;
    } else {                                   // the last, partial macro-step (K is a multiple of 8)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) f.w[t][j] = (kb + 8 * j + 8 <= K) ? *(const u32x4 *)(wrow[t] + kb + 8 * j) : zero;
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                f.x[m][j] = (xvalid[m] && kb + 8 * j + 8 <= K) ? *(const u32x4 *)(xrow[m] + kb + 8 * j) : zero;
    }
}

template <int NT, int MT>
__device__ __forceinline__ void mul_frag(const Frag<NT, MT> &f, f32x4 (&acc)[NT][MT]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[t][m] = mfma16(f.w[t][j], f.x[m][j], acc[t][m]);
}

template <int NT, int MT, int EPI, int SK_WAVES, bool PACKED>
__global__ void __launch_bounds__(SK_WAVES *WAVE)
gemm_skinny_kernel(const bf16_t *__restrict__ X, int ldx, const bf16_t *__restrict__ W, int ldw, void *__restrict__ Y,
                   int ldy, int M, int N, int K, SkinnyExtra ex) {
    __shared__ float red[SK_WAVES][NT * MT * 4][WAVE];
    __shared__ float row_scale[16 * MT];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int l16 = lane & 15, grp = lane >> 4;
    // the rows of W of tile t: for SwiGLU tile 0 are gate rows, tile 1 the up rows N/2 further
    const int n_out = EPI == EPI_SWIGLU ? N / 2 : N;                 // width of Y
    // SwiGLU: the first NT/2 tiles are gate rows, the other NT/2 the up rows N/2 further
    const int n0 = blockIdx.x * 16 * (EPI == EPI_SWIGLU ? NT / 2 : NT);
    // q/k/v with rotation: workgroup b has, of head b / (head_dim/32), the dims 16 c .. and head_dim/2 + 16 c ..
    const int rope_head = EPI == EPI_QKV_ROPE ? blockIdx.x / (ex.head_dim / 32) : 0;
    const int rope_c = EPI == EPI_QKV_ROPE ? blockIdx.x % (ex.head_dim / 32) : 0;
    const bf16_t *wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int half = t / (NT / 2 > 0 ? NT / 2 : 1);              // 0: gate tiles, 1: up tiles (SwiGLU)
        int row = EPI == EPI_SWIGLU ? n0 + 16 * (t % (NT / 2 > 0 ? NT / 2 : 1)) + l16 + half * n_out : n0 + 16 * t + l16;
        if (EPI == EPI_QKV_ROPE) row = rope_head * ex.head_dim + t * (ex.head_dim / 2) + 16 * rope_c + l16;
        const int limit = EPI == EPI_SWIGLU ? (half + 1) * n_out : N;
        row = row < limit ? row : limit - 1;                          // a row beyond the end is read, not stored
        wrow[t] = PACKED ? W + ((size_t)(row / 16) * (K / 128)) * 2048 + (size_t)lane * 8   // (the tile of the row)
                           : W + (size_t)row * ldw;
    }
    const bf16_t *xrow[MT];
    bool xvalid[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        xvalid[m] = 16 * m + l16 < M;
        xrow[m] = X + (size_t)(xvalid[m] ? 16 * m + l16 : 0) * ldx;
    }
    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = f32x4{0.f, 0.f, 0.f, 0.f};

    // The rows' factors, by the last wave before it starts on its share of K.  Lane group g adds
    // the g-th quarter of a row's shares, eight 16-byte loads in flight at a time (one load after
    // the other would hold the wave back for tens of microseconds); the quarters' sums are added
    // in the order of the shuffles.  Always the same order: no dependence on timing.
    if (EPI != EPI_ADD_NORM && ex.sumsq_in != nullptr && wave == SK_WAVES - 1) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int tok = 16 * m + l16;
            const float *p = ex.sumsq_in + (size_t)(tok < M ? tok : 0) * ex.n_in;
            float ss = 0.f;
            if ((ex.n_in & 15) == 0) {
                const int q4 = ex.n_in / 16;                       // float4s in a quarter
                const f32x4 *p4 = (const f32x4 *)p + grp * q4;
                for (int i = 0; i < q4; i += 8) {
                    f32x4 v[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = p4[i + e < q4 ? i + e : q4 - 1];
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (i + e < q4) ss += (v[e][0] + v[e][1]) + (v[e][2] + v[e][3]);
                }
            } else {
                for (int i = grp; i < ex.n_in; i += 4) ss += p[i];
            }
            ss += __shfl_xor(ss, 16, WAVE);
            ss += __shfl_xor(ss, 32, WAVE);
            if (grp == 0) row_scale[tok] = rsqrtf(ss / (float)ex.norm_width + ex.eps);
        }
    }

    // A ring of STAGES macro-steps in flight per wave: with few workgroups per compute unit
    // (small N) this is what keeps enough bytes on their way from HBM.
    constexpr int STAGES = NT * MT == 1 ? 4 : (NT * MT == 2 ? 3 : 2);
    const int nsteps = (K + 127) / 128;
    Frag<NT, MT> f[STAGES];
    int s = wave;
#pragma unroll
    for (int i = 0; i < STAGES; ++i)
        if (s + i * SK_WAVES < nsteps) load_frag<NT, MT, PACKED>(f[i], wrow, xrow, xvalid, s + i * SK_WAVES, grp, K);
    for (; s < nsteps; s += STAGES * SK_WAVES) {
#pragma unroll
        for (int i = 0; i < STAGES; ++i) {
            const int cur = s + i * SK_WAVES;
            if (cur < nsteps) {
                mul_frag<NT, MT>(f[i], acc);
                if (cur + STAGES * SK_WAVES < nsteps)
                    load_frag<NT, MT, PACKED>(f[i], wrow, xrow, xvalid, cur + STAGES * SK_WAVES, grp, K);
            }
        }
    }
    // ---- the waves' sums, added in the order 0, 1, 2, ...
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave][(t * MT + m) * 4 + r][lane] = acc[t][m][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = (t * MT + m) * 4 + r;
                float sum = red[0][i][lane];
#pragma unroll
                for (int w = 1; w < SK_WAVES; ++w) sum += red[w][i][lane];
                acc[t][m][r] = sum;
            }
    // ---- epilogue: the lane holds, per tile, features 4 grp + r of token 16 m + l16
    if (EPI != EPI_ADD_NORM && ex.sumsq_in != nullptr) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float rs = row_scale[16 * m + l16];
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][m][r] *= rs;
        }
    }
    if (EPI == EPI_QKV_ROPE) {
        // the lane holds dims i = 16 c + 4 grp + r (tile 0) and i + head_dim/2 (tile 1) of token 16 m + l16
        const int dh = ex.head_dim, half_dim = dh / 2;
        const bool is_q = rope_head < ex.heads, is_k = !is_q && rope_head < ex.heads + ex.kv_heads;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int tok = 16 * m + l16;
            if (tok >= M) continue;
            const int pos = ex.positions[tok];
            const bool in_table = pos >= 0 && pos < ex.max_pos;
            const int slot = ex.slots ? ex.slots[tok] : -1;
            bf16_t *pg = nullptr;
            int place = 0;
            if (!is_q && slot >= 0) {
                pg = ex.cache + (size_t)(slot / ex.page) * kv_page_elems(ex.kv_heads, dh, ex.page);
                place = slot % ex.page;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 16 * rope_c + 4 * grp + r;
                // rounded to bfloat16 before the rotation, as the product's plain epilogue stores them for
                // the rotation kernel: a token's query and key are the same bits whichever way they are made
                float a = to_f32(from_f32<bf16_t>(acc[0][m][r])), b = to_f32(from_f32<bf16_t>(acc[NT - 1][m][r]));
                if (is_q || is_k) {
                    float c = __uint_as_float(0x7fc00000u), sn = c;         // a position outside the table gives NaN
                    if (in_table) { c = ex.cos_t[(size_t)pos * half_dim + i]; sn = ex.sin_t[(size_t)pos * half_dim + i]; }
                    float ra, rb;
                    rotate_pair(a, b, c, sn, ra, rb);
                    a = ra; b = rb;
                }
                const bf16_t va = from_f32<bf16_t>(a), vb = from_f32<bf16_t>(b);
                if (is_q) {
                    bf16_t *qo = ex.q_out + (size_t)tok * ex.ldq + (size_t)rope_head * dh;
                    qo[i] = va;
                    qo[i + half_dim] = vb;
                } else if (pg) {
                    if (is_k) {
                        const int kvh = rope_head - ex.heads;
                        pg[kv_key_offset(kvh, place, i, dh, ex.page)] = va;
                        pg[kv_key_offset(kvh, place, i + half_dim, dh, ex.page)] = vb;
                    } else {
                        const int kvh = rope_head - ex.heads - ex.kv_heads;
                        pg[kv_value_offset(ex.kv_heads, kvh, place, i, dh, ex.page)] = va;
                        pg[kv_value_offset(ex.kv_heads, kvh, place, i + half_dim, dh, ex.page)] = vb;
                    }
                }
            }
        }
        return;
    }
    if (EPI == EPI_ADD_NORM) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int tok = 16 * m + l16;
            float ss = 0.f;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + 16 * t + 4 * grp + r;
                    if (tok >= M || n >= N) continue;
                    float *res = (float *)Y + (size_t)tok * ldy + n;
                    const float xn = *res + acc[t][m][r];
                    *res = xn;
                    ss += xn * xn;
                    const float wn = ex.norm_w_type == LCU_F32 ? ((const float *)ex.norm_w)[n] : to_f32(((const bf16_t *)ex.norm_w)[n]);
                    ex.h_out[(size_t)tok * ex.ldh + n] = from_f32<bf16_t>(xn * wn);
                }
            ss += __shfl_xor(ss, 16, WAVE);               // every lane takes part: the others bring zero
            ss += __shfl_xor(ss, 32, WAVE);
            if (grp == 0 && tok < M) ex.sumsq_out[(size_t)tok * gridDim.x + blockIdx.x] = ss;
        }
        return;
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int tok = 16 * m + l16;
        if (tok >= M) continue;
        if (EPI == EPI_SWIGLU) {
#pragma unroll
            for (int t = 0; t < NT / 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + 16 * t + 4 * grp + r;
                    if (n >= n_out) continue;
                    const float gate = acc[t][m][r], up = acc[t + NT / 2][m][r];
                    const float sig = 1.0f / (1.0f + expf(-gate));
                    ((bf16_t *)Y)[(size_t)tok * ldy + n] = from_f32<bf16_t>(gate * sig * up);
                }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + 16 * t + 4 * grp + r;
                    if (n >= N) continue;
                    const size_t at = (size_t)tok * ldy + n;
                    if (EPI == EPI_BF16) ((bf16_t *)Y)[at] = from_f32<bf16_t>(acc[t][m][r]);
                    else if (EPI == EPI_F32) ((float *)Y)[at] = acc[t][m][r];
                    else ((float *)Y)[at] += acc[t][m][r];
                }
        }
    }
}

template <int NT, int MT, int WAVES>
static int launch_epi(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K, int epi,
                      int packed, const SkinnyExtra &ex, hipStream_t stream) {
    dim3 block(WAVES * WAVE);
    const dim3 grid((N + 16 * NT - 1) / (16 * NT));
#define GO(E)                                                                                                                      \
    do {                                                                                                                           \
        if (packed) gemm_skinny_kernel<NT, MT, E, WAVES, true><<<grid, block, 0, stream>>>((const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, ex); \
        else gemm_skinny_kernel<NT, MT, E, WAVES, false><<<grid, block, 0, stream>>>((const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, ex);       \
    } while (0)
    switch (epi) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    case EPI_ADD_F32: GO(EPI_ADD_F32); break;
    case EPI_ADD_NORM:
        if constexpr (MT <= 2 && NT <= 2) { GO(EPI_ADD_NORM); break; }      // made for decoding: at most 32 rows
        return LCU_UNSUPPORTED;
    case EPI_QKV_ROPE:
        if constexpr (MT <= 2 && NT == 2) {
            const dim3 rgrid((ex.heads + 2 * ex.kv_heads) * (ex.head_dim / 32));
            if (packed) gemm_skinny_kernel<NT, MT, EPI_QKV_ROPE, WAVES, true><<<rgrid, block, 0, stream>>>(
                (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, ex);
            else gemm_skinny_kernel<NT, MT, EPI_QKV_ROPE, WAVES, false><<<rgrid, block, 0, stream>>>(
                (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, ex);
            break;
        }
        return LCU_UNSUPPORTED;
    default: return LCU_BAD_ARGUMENT;
    }
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

template <int NT, int MT, int WAVES>
static int launch_swiglu(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K,
                         int packed, const SkinnyExtra &ex, hipStream_t stream) {
    const int groups = (N / 2 + 8 * NT - 1) / (8 * NT);
    if (packed) gemm_skinny_kernel<NT, MT, EPI_SWIGLU, WAVES, true><<<dim3(groups), dim3(WAVES * WAVE), 0, stream>>>(
        (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, ex);
    else gemm_skinny_kernel<NT, MT, EPI_SWIGLU, WAVES, false><<<dim3(groups), dim3(WAVES * WAVE), 0, stream>>>(
        (const bf16_t *)X, ldx, (const bf16_t *)W, ldw, Y, ldy, M, N, K, ex);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// X: [M, K] bfloat16 rows ldx apart; W: [N, K] bfloat16 rows ldw apart; Y: [M, N] rows ldy
// apart (for the SwiGLU epilogue [M, N/2]: W holds N/2 gate rows, then N/2 up rows).
// M <= 32; K, ldx and ldw multiples of 8 (16-byte loads); tiles: output tiles of 16
// features per workgroup (1, 2 or 4; more tiles reuse X more, fewer give more workgroups);
// waves: 4 or 8 waves share a workgroup's K.
static int skinny_bf16(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K, int epilogue,
                       int tiles, int waves, int packed, const SkinnyExtra &ex, hipStream_t stream) {
    if (M <= 0 || N <= 0) return LCU_OK;
    // a packed weight is whole blocks of 16 rows x 128 k (and for SwiGLU each half is)
    if (packed && (K % 128 || N % 16 || (epilogue == EPI_SWIGLU && N % 32))) return LCU_BAD_ARGUMENT;
    if (M > 32 || K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || ldw < K) return LCU_BAD_ARGUMENT;
    if (waves != 4 && waves != 8) return LCU_BAD_ARGUMENT;
    const int mt = (M + 15) / 16;
    if (epilogue == EPI_SWIGLU) {
        if (N % 2 || ldy < N / 2) return LCU_BAD_ARGUMENT;
        // tiles: gate and up tiles together (2: one of each, 4: two of each)
#define SW(NT_, MT_) return waves == 8 ? launch_swiglu<NT_, MT_, 8>(X, ldx, W, ldw, Y, ldy, M, N, K, packed, ex, stream) \
                                       : launch_swiglu<NT_, MT_, 4>(X, ldx, W, ldw, Y, ldy, M, N, K, packed, ex, stream)
        if (tiles == 4 && mt <= 2) {
            if (mt == 1) SW(4, 1);
            SW(4, 2);
        }
        if (mt == 1) SW(2, 1);
        SW(2, 2);
#undef SW
    }
    if (ldy < N) return LCU_BAD_ARGUMENT;
#define EP(NT_, MT_) return waves == 8 ? launch_epi<NT_, MT_, 8>(X, ldx, W, ldw, Y, ldy, M, N, K, epilogue, packed, ex, stream) \
                                       : launch_epi<NT_, MT_, 4>(X, ldx, W, ldw, Y, ldy, M, N, K, epilogue, packed, ex, stream)
#define PICK(NT_)          \
    if (mt == 1) EP(NT_, 1); \
    EP(NT_, 2);
    if (tiles == 1) { PICK(1) }
    if (tiles == 2) { PICK(2) }
    if (tiles == 4) { PICK(4) }
#undef PICK
#undef EP
    return LCU_BAD_ARGUMENT;
}

LCU_API int lcu_gemm_skinny_bf16(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K,
                                 int epilogue, int tiles, int waves, int w_packed, hipStream_t stream) {
    if (epilogue == EPI_ADD_NORM) return LCU_BAD_ARGUMENT;
    const SkinnyExtra none = {};
    return skinny_bf16(X, ldx, W, ldw, Y, ldy, M, N, K, epilogue, tiles, waves, w_packed, none, stream);
}

// The product that ends a branch, the residual sum and the next norm's weight in one kernel:
// res[M, N] (float32, rows ldres apart) += X W^T; h_out[M, N] = bfloat16(res * norm_w), not yet
// normalised; sumsq_out[M][ceil(N / (16 tiles))] = each workgroup's share of the rows' sums of
// squares.  At most 32 rows, tiles 1 or 2.
LCU_API int lcu_gemm_skinny_bf16_add_norm(const void *X, int ldx, const void *W, int ldw, float *res, int ldres, int M, int N,
                                          int K, const void *norm_w, int norm_w_type, void *h_out, int ldh, float *sumsq_out,
                                          int sumsq_cols, int tiles, int waves, int w_packed, hipStream_t stream) {
    if (M > 32 || (tiles != 1 && tiles != 2) || !res || !norm_w || !h_out || !sumsq_out || ldh < N || ldres < N ||
        (norm_w_type != LCU_F32 && norm_w_type != LCU_BF16) || sumsq_cols != (N + 16 * tiles - 1) / (16 * tiles))
        return LCU_BAD_ARGUMENT;
    SkinnyExtra ex = {};
    ex.norm_w = norm_w; ex.norm_w_type = norm_w_type; ex.h_out = (bf16_t *)h_out; ex.ldh = ldh; ex.sumsq_out = sumsq_out;
    return skinny_bf16(X, ldx, W, ldw, res, ldres, M, N, K, EPI_ADD_NORM, tiles, waves, w_packed, ex, stream);
}

// A product whose rows of X wait for their normalisation: row i of the product is multiplied by
// rsqrt(sum(sumsq_in[i][0 .. n_in)) / norm_width + eps) before the epilogue (not EPI_ADD_NORM).
LCU_API int lcu_gemm_skinny_bf16_scaled(const void *X, int ldx, const void *W, int ldw, void *Y, int ldy, int M, int N, int K,
                                        int epilogue, int tiles, int waves, int w_packed, const float *sumsq_in, int n_in,
                                        int norm_width, float eps, hipStream_t stream) {
    if (epilogue == EPI_ADD_NORM || !sumsq_in || n_in <= 0 || norm_width <= 0) return LCU_BAD_ARGUMENT;
    SkinnyExtra ex = {};
    ex.sumsq_in = sumsq_in; ex.n_in = n_in; ex.norm_width = norm_width; ex.eps = eps;
    return skinny_bf16(X, ldx, W, ldw, Y, ldy, M, N, K, epilogue, tiles, waves, w_packed, ex, stream);
}


// The q, k and v projections with the rotation and the cache write in the epilogue.  W: [(heads +
// 2 kv_heads) * head_dim, K] (q heads, then k heads, then v heads).  q_out: [M, heads * head_dim]
// rows ldq apart takes the rotated queries; the rotated keys and the values go to cache (this
// layer's pages, laid out as kv_layout.h says) at slots[m] (page * page_size + place; -1: nothing
// is stored).  cos_t, sin_t: [max_pos, head_dim / 2] float32; pairs are (i, i + head_dim / 2).
// At most 32 rows; head_dim a multiple of 32.  sumsq_in (may be null): the rows of X wait for
// their normalisation, as in lcu_gemm_skinny_bf16_scaled.
LCU_API int lcu_gemm_skinny_bf16_qkv_rope(const void *X, int ldx, const void *W, int ldw, int M, int K, void *q_out, int ldq,
                                          const int *positions, const int *slots, const float *cos_t, const float *sin_t,
                                          int max_pos, void *cache, int heads, int kv_heads, int head_dim, int page,
                                          int waves, int w_packed, const float *sumsq_in, int n_in, int norm_width, float eps,
                                          hipStream_t stream) {
    if (M <= 0) return LCU_OK;
    if (M > 32 || heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim % 32 || page <= 0 || page % 8 || !q_out ||
        !positions || !cos_t || !sin_t || max_pos <= 0 || !cache || ldq < heads * head_dim ||
        (sumsq_in && (n_in <= 0 || norm_width <= 0)))
        return LCU_BAD_ARGUMENT;
    SkinnyExtra ex = {};
    ex.sumsq_in = sumsq_in; ex.n_in = n_in; ex.norm_width = norm_width; ex.eps = eps;
    ex.positions = positions; ex.slots = slots; ex.cos_t = cos_t; ex.sin_t = sin_t; ex.max_pos = max_pos;
    ex.cache = (bf16_t *)cache; ex.q_out = (bf16_t *)q_out; ex.ldq = ldq;
    ex.heads = heads; ex.kv_heads = kv_heads; ex.head_dim = head_dim; ex.page = page;
    const int N = (heads + 2 * kv_heads) * head_dim;
    return skinny_bf16(X, ldx, W, ldw, q_out, N, M, N, K, EPI_QKV_ROPE, 2, waves, w_packed, ex, stream);
}


// ============================================================================ float32
// The same weight-streaming layout for float32 operands, with v_mfma_f32_16x16x4_f32: a true
// 32-bit matrix product (32-bit multiplies and adds; no reduced-precision mode).  A lane's
// 16-byte load holds four k of its row, one per instruction.  K goes in macro-steps of 64; the
// waves of a workgroup take macro-steps in turn and their sums are added in a fixed order, so
// a token's result depends on K and the number of waves only: not on M, not on which tile of
// 64 tokens (grid.y) it is in, not on the other tokens.
constexpr int F32_WAVES = 8;

template <int MT>
struct FragF32 {
    f32x4 w[4];
    f32x4 x[MT][4];
};

template <int MT>
__device__ __forceinline__ void load_frag_f32(FragF32<MT> &f, const float *wrow, const float *const (&xrow)[MT],
                                              const bool (&xvalid)[MT], int s, int grp, int K) {
    const int kb = 64 * s + 16 * grp;
    const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const bool in = kb + 4 * j + 4 <= K;                // K is a multiple of 4
        f.w[j] = in ? *(const f32x4 *)(wrow + kb + 4 * j) : zero;
#pragma unroll
        for (int m = 0; m < MT; ++m) f.x[m][j] = (in && xvalid[m]) ? *(const f32x4 *)(xrow[m] + kb + 4 * j) : zero;
    }
}

template <int MT>
__global__ void __launch_bounds__(F32_WAVES *WAVE)
gemm_skinny_f32_kernel(const float *__restrict__ X, int ldx, const float *__restrict__ W, int ldw, float *__restrict__ Y,
                       int ldy, int M, int N, int K, int accumulate) {
    __shared__ float red[F32_WAVES][MT * 4][WAVE];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int l16 = lane & 15, grp = lane >> 4;
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16 * MT;
    int row = n0 + l16;
    row = row < N ? row : N - 1;                            // a row beyond the end is read, not stored
    const float *wrow = W + (size_t)row * ldw;
    const float *xrow[MT];
    bool xvalid[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        xvalid[m] = m0 + 16 * m + l16 < M;
        xrow[m] = X + (size_t)(xvalid[m] ? m0 + 16 * m + l16 : 0) * ldx;
    }
    f32x4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int nsteps = (K + 63) / 64;
    FragF32<MT> fa, fb;
    int s = wave;
    if (s < nsteps) load_frag_f32<MT>(fa, wrow, xrow, xvalid, s, grp, K);
    for (; s < nsteps; s += 2 * F32_WAVES) {
        const bool has_b = s + F32_WAVES < nsteps;
        if (has_b) load_frag_f32<MT>(fb, wrow, xrow, xvalid, s + F32_WAVES, grp, K);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int m = 0; m < MT; ++m) acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa.w[j][e], fa.x[m][j][e], acc[m], 0, 0, 0);
        if (s + 2 * F32_WAVES < nsteps) load_frag_f32<MT>(fa, wrow, xrow, xvalid, s + 2 * F32_WAVES, grp, K);
        if (has_b) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int m = 0; m < MT; ++m) acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(fb.w[j][e], fb.x[m][j][e], acc[m], 0, 0, 0);
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][m * 4 + r][lane] = acc[m][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int tok = m0 + 16 * m + l16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float sum = red[0][m * 4 + r][lane];
#pragma unroll
            for (int w = 1; w < F32_WAVES; ++w) sum += red[w][m * 4 + r][lane];
            const int n = n0 + 4 * grp + r;
            if (tok < M && n < N) {
                float *y = Y + (size_t)tok * ldy + n;
                *y = accumulate ? *y + sum : sum;
            }
        }
    }
}

// X: [M, K] float32, W: [N, K] float32, Y: [M, N] float32 (accumulate: Y += X W^T).  Any M
// (tiles of 64 tokens; W is read once per tile); K, ldx, ldw multiples of 4.
LCU_API int lcu_gemm_skinny_f32(const float *X, int ldx, const float *W, int ldw, float *Y, int ldy, int M, int N,
                                int K, int accumulate, hipStream_t stream) {
    if (M <= 0 || N <= 0) return LCU_OK;
    if (K <= 0 || K % 4 || ldx % 4 || ldw % 4 || ldx < K || ldw < K || ldy < N) return LCU_BAD_ARGUMENT;
    const dim3 block(F32_WAVES * WAVE);
    if (M <= 16) {
        gemm_skinny_f32_kernel<1><<<dim3((N + 15) / 16, 1), block, 0, stream>>>(X, ldx, W, ldw, Y, ldy, M, N, K, accumulate);
    } else {
        const int tiles = (M + 63) / 64;
        if (tiles > 65535) return LCU_BAD_ARGUMENT;
        gemm_skinny_f32_kernel<4><<<dim3((N + 15) / 16, tiles), block, 0, stream>>>(X, ldx, W, ldw, Y, ldy, M, N, K, accumulate);
    }
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
