// Row-wise kernels: embedding gather, row gather, RMS norm fused with the residual
// sum, SwiGLU, residual add.  Sums, the norm and the activation are computed in
// 32-bit whatever the storage type.
#include "common.h"

// ---------------------------------------------------------------- embedding gather
// out[i, :] = table[ids[i], :].  An id outside the table writes NaN into the row
// (the host checks ids before; this keeps a bad id from reading out of bounds).
template <class TT, class TO>
__global__ void embedding_gather_kernel(TO *__restrict__ out, const TT *__restrict__ table,
                                        const int *__restrict__ ids, int d, int vocab) {
    const int row = blockIdx.x;
    const int id = ids[row];
    TO *o = out + (size_t)row * d;
    if (id < 0 || id >= vocab) {
        for (int c = threadIdx.x; c < d; c += blockDim.x) o[c] = from_f32<TO>(__uint_as_float(0x7fc00000u));
        return;
    }
    const TT *t = table + (size_t)id * d;
    if (d % 8 == 0 && ((size_t)t % (8 * sizeof(TT))) == 0 && ((size_t)o % (8 * sizeof(TO))) == 0) {
        // eight neighbouring elements per load (a row is read once, from memory: few, wide loads)
        struct alignas(8 * sizeof(TT)) In8 { TT v[8]; };
        struct alignas(8 * sizeof(TO)) Out8 { TO v[8]; };
        for (int c = threadIdx.x * 8; c < d; c += blockDim.x * 8) {
            const In8 in = *(const In8 *)(t + c);
            Out8 res;
#pragma unroll
            for (int e = 0; e < 8; ++e) res.v[e] = from_f32<TO>(to_f32(in.v[e]));
            *(Out8 *)(o + c) = res;
        }
        return;
    }
    for (int c = threadIdx.x; c < d; c += blockDim.x) o[c] = from_f32<TO>(to_f32(t[c]));
}

LCU_API int lcu_embedding_gather(void *out, int out_type, const void *table, int table_type,
                                 const int *ids, int n, int d, int vocab, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || vocab <= 0) return LCU_BAD_ARGUMENT;
    dim3 grid(n), block(256);
#define GO(TT, TO) embedding_gather_kernel<TT, TO><<<grid, block, 0, stream>>>((TO *)out, (const TT *)table, ids, d, vocab)
    if (table_type == LCU_F32 && out_type == LCU_F32) GO(float, float);
    else if (table_type == LCU_BF16 && out_type == LCU_F32) GO(bf16_t, float);
    else if (table_type == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t);
    else if (table_type == LCU_F32 && out_type == LCU_BF16) GO(float, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- row gather
template <class T>
__global__ void gather_rows_kernel(T *__restrict__ out, const T *__restrict__ x,
                                   const int *__restrict__ rows, int d, int n_src) {
    const int r = rows[blockIdx.x];
    T *o = out + (size_t)blockIdx.x * d;
    if (r < 0 || r >= n_src) {
        for (int c = threadIdx.x; c < d; c += blockDim.x) o[c] = from_f32<T>(__uint_as_float(0x7fc00000u));
        return;
    }
    const T *s = x + (size_t)r * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) o[c] = s[c];
}

LCU_API int lcu_gather_rows(void *out, const void *x, int type, const int *rows, int n_out, int d,
                            int n_src, hipStream_t stream) {
    if (n_out <= 0) return LCU_OK;
    if (d <= 0) return LCU_BAD_ARGUMENT;
    dim3 grid(n_out), block(256);
    if (type == LCU_F32) gather_rows_kernel<float><<<grid, block, 0, stream>>>((float *)out, (const float *)x, rows, d, n_src);
    else if (type == LCU_BF16) gather_rows_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t *)out, (const bf16_t *)x, rows, d, n_src);
    else return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- RMS norm (+ residual sum)
// One block per row.  If `delta` is given: x += delta first (in 32-bit, written back
// when x is 32-bit: x is then the residual stream); delta may be `planes` planes [n, d],
// `plane_stride` elements apart (a product's partial sums over slices of K), which are added
// one after the other in the order of the planes.  Then
//   y = x * rsqrt(sum(x^2)/d + eps) * w        (32-bit, one rounding at the store)
// The order of the sum depends on d and the block size only, not on the batch.
template <class TX, class TD, class TW, class TO>
__global__ void rmsnorm_kernel(TX *__restrict__ x, const TD *__restrict__ delta, const TW *__restrict__ w,
                               TO *__restrict__ out, int d, float eps, int write_back, int planes, size_t plane_stride) {
    __shared__ float scratch[16];
    TX *xr = x + (size_t)blockIdx.x * d;
    const TD *dr = delta ? delta + (size_t)blockIdx.x * d : nullptr;
    float acc = 0.f;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        float v = to_f32(xr[c]);
        if (dr) {
            for (int p = 0; p < planes; ++p) v += to_f32(dr[p * plane_stride + c]);
            if (write_back) xr[c] = from_f32<TX>(v);
        }
        acc += v * v;
    }
    const float total = block_sum(acc, scratch);
    const float rms = rsqrtf(total / (float)d + eps);
    TO *o = out + (size_t)blockIdx.x * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        float v = to_f32(xr[c]);
        if (dr && !write_back)
            for (int p = 0; p < planes; ++p) v += to_f32(dr[p * plane_stride + c]);
        o[c] = from_f32<TO>(rms * v * to_f32(w[c]));
    }
}

// The same for rows of up to 8192 elements whose width is a multiple of 4: one read of
// the row (four elements per load), the row kept in registers between the sum and the
// scaling.  The row is dealt to 1024 virtual threads, two loads each; a block has 1024
// threads (few rows leave most of the chip idle: what counts then is how many loads a row has
// in flight) or 256 that play four virtual threads each (many rows: fewer, longer-lived waves
// stream faster).  The sums are added as the 1024 threads would add them, wave by wave, so
// the result does not depend on the block's size, only on d.  The planes are loaded four at
// a time.
constexpr int NORM_VTHREADS = 1024, NORM_ITEMS = 2;

template <class T> struct alignas(4 * sizeof(T)) Vec4 { T v[4]; };

template <int THREADS, class TX, class TD, class TW, class TO>
__global__ void __launch_bounds__(THREADS)
rmsnorm_fast_kernel(TX *__restrict__ x, const TD *__restrict__ delta, const TW *__restrict__ w, TO *__restrict__ out,
                    int d, float eps, int write_back, int planes, size_t plane_stride) {
    constexpr int PLAY = NORM_VTHREADS / THREADS;           // virtual threads per thread
    __shared__ float scratch[NORM_VTHREADS / WAVE];
    TX *xr = x + (size_t)blockIdx.x * d;
    const TD *dr = delta ? delta + (size_t)blockIdx.x * d : nullptr;
    float v[PLAY][NORM_ITEMS][4];
#pragma unroll
    for (int j = 0; j < PLAY; ++j) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NORM_ITEMS; ++i) {
            const int c = (i * NORM_VTHREADS + j * THREADS + threadIdx.x) * 4;
            if (c < d) {
                const Vec4<TX> xv = *(const Vec4<TX> *)(xr + c);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[j][i][e] = to_f32(xv.v[e]);
                if (dr) {
                    for (int p0 = 0; p0 < planes; p0 += 4) {
                        Vec4<TD> dv[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) dv[q] = *(const Vec4<TD> *)(dr + (p0 + q < planes ? p0 + q : p0) * plane_stride + c);
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            if (p0 + q < planes) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) v[j][i][e] += to_f32(dv[q].v[e]);
                            }
                    }
                    Vec4<TX> back;
#pragma unroll
                    for (int e = 0; e < 4; ++e) back.v[e] = from_f32<TX>(v[j][i][e]);
                    if (write_back) *(Vec4<TX> *)(xr + c) = back;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) acc += v[j][i][e] * v[j][i][e];
            }
        }
        // the wave of the 1024 threads that these virtual threads are
        acc = wave_sum(acc);
        if ((threadIdx.x & (WAVE - 1)) == 0) scratch[j * (THREADS / WAVE) + threadIdx.x / WAVE] = acc;
    }
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < NORM_VTHREADS / WAVE; ++k) total += scratch[k];
    const float rms = rsqrtf(total / (float)d + eps);
    TO *o = out + (size_t)blockIdx.x * d;
#pragma unroll
    for (int j = 0; j < PLAY; ++j)
#pragma unroll
        for (int i = 0; i < NORM_ITEMS; ++i) {
            const int c = (i * NORM_VTHREADS + j * THREADS + threadIdx.x) * 4;
            if (c < d) {
                const Vec4<TW> wv = *(const Vec4<TW> *)(w + c);
                Vec4<TO> ov;
#pragma unroll
                for (int e = 0; e < 4; ++e) ov.v[e] = from_f32<TO>(rms * v[j][i][e] * to_f32(wv.v[e]));
                *(Vec4<TO> *)(o + c) = ov;
            }
        }
}

template <class TX, class TD, class TO>
static int rmsnorm_w(void *x, const void *delta, const void *w, int w_type, void *out, int n, int d, float eps,
                     int write_back, hipStream_t stream, int planes = 1, size_t plane_stride = 0) {
    dim3 grid(n), block(d >= 2048 ? 512 : 256);
    if (d % 4 == 0 && d <= NORM_VTHREADS * NORM_ITEMS * 4) {
#define FAST(T_, TW_) rmsnorm_fast_kernel<T_, TX, TD, TW_, TO><<<grid, dim3(T_), 0, stream>>>((TX *)x, (const TD *)delta, (const TW_ *)w, (TO *)out, d, eps, write_back, planes, plane_stride)
        const bool few = n <= 192;        // (measured with four planes: steps of 160 and 192 rows 2 % faster with 1024 threads, of 256 rows 1 % slower)
        if (w_type == LCU_F32) {
            if (few) FAST(1024, float); else FAST(256, float);
        } else if (w_type == LCU_BF16) {
            if (few) FAST(1024, bf16_t); else FAST(256, bf16_t);
        } else {
            return LCU_BAD_ARGUMENT;
        }
#undef FAST
        LCU_LAUNCH_CHECK();
        return LCU_OK;
    }
    if (w_type == LCU_F32)
        rmsnorm_kernel<TX, TD, float, TO><<<grid, block, 0, stream>>>((TX *)x, (const TD *)delta, (const float *)w, (TO *)out, d, eps, write_back, planes, plane_stride);
    else if (w_type == LCU_BF16)
        rmsnorm_kernel<TX, TD, bf16_t, TO><<<grid, block, 0, stream>>>((TX *)x, (const TD *)delta, (const bf16_t *)w, (TO *)out, d, eps, write_back, planes, plane_stride);
    else
        return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// x: [n, d] of x_type (read; written when write_back and delta are set), delta: [n, d] of
// act_type or null, out: [n, d] of act_type.
LCU_API int lcu_rmsnorm(void *x, int x_type, const void *delta, const void *w, int w_type, void *out,
                        int act_type, int n, int d, float eps, int write_back, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0) return LCU_BAD_ARGUMENT;
    if (x_type == LCU_F32 && act_type == LCU_F32) return rmsnorm_w<float, float, float>(x, delta, w, w_type, out, n, d, eps, write_back, stream);
    if (x_type == LCU_F32 && act_type == LCU_BF16) return rmsnorm_w<float, bf16_t, bf16_t>(x, delta, w, w_type, out, n, d, eps, write_back, stream);
    if (x_type == LCU_BF16 && act_type == LCU_BF16) return rmsnorm_w<bf16_t, bf16_t, bf16_t>(x, delta, w, w_type, out, n, d, eps, write_back, stream);
    return LCU_BAD_ARGUMENT;
}

// The same with the branch's output as `planes` float32 planes [n, d], one after the other:
// x (float32) += plane 0 + plane 1 + ... (in this order), then the norm.  d a multiple of 4.
LCU_API int lcu_rmsnorm_planes(float *x, const float *planes_ptr, int planes, const void *w, int w_type, void *out,
                               int act_type, int n, int d, float eps, int write_back, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || d % 4 || planes <= 0 || !planes_ptr) return LCU_BAD_ARGUMENT;
    const size_t stride = (size_t)n * d;
    if (act_type == LCU_F32) return rmsnorm_w<float, float, float>(x, planes_ptr, w, w_type, out, n, d, eps, write_back, stream, planes, stride);
    if (act_type == LCU_BF16) return rmsnorm_w<float, float, bf16_t>(x, planes_ptr, w, w_type, out, n, d, eps, write_back, stream, planes, stride);
    return LCU_BAD_ARGUMENT;
}

// ---------------------------------------------------------------- residual add: x (f32) += delta
template <class TD>
__global__ void residual_add_kernel(float *__restrict__ x, const TD *__restrict__ delta, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) x[i] += to_f32(delta[i]);
}

LCU_API int lcu_residual_add(float *x, const void *delta, int delta_type, long long total, hipStream_t stream) {
    if (total <= 0) return LCU_OK;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    if (delta_type == LCU_F32) residual_add_kernel<float><<<grid, block, 0, stream>>>(x, (const float *)delta, (size_t)total);
    else if (delta_type == LCU_BF16) residual_add_kernel<bf16_t><<<grid, block, 0, stream>>>(x, (const bf16_t *)delta, (size_t)total);
    else return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- SwiGLU
// out[r, c] = gate * (1 / (1 + exp(-gate))) * up with gate = gu[r, c], up = gu[r, di + c].
template <class T>
__global__ void swiglu_kernel(T *__restrict__ out, const T *__restrict__ gu, int di) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= di) return;
    const size_t r = blockIdx.y;
    const float gate = to_f32(gu[r * 2 * di + c]);
    const float up = to_f32(gu[r * 2 * di + di + c]);
    const float sig = 1.0f / (1.0f + expf(-gate));
    out[r * di + c] = from_f32<T>(gate * sig * up);
}

// The same, eight neighbouring columns per thread (16-byte loads of bfloat16, 32-byte of
// float32); for widths that are multiples of 8.
template <class T> struct alignas(8 * sizeof(T)) Vec8 { T v[8]; };

template <class T>
__global__ void swiglu_vec8_kernel(T *__restrict__ out, const T *__restrict__ gu, int di) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= di) return;
    const size_t r = blockIdx.y;
    const Vec8<T> g = *(const Vec8<T> *)(gu + r * 2 * di + c);
    const Vec8<T> u = *(const Vec8<T> *)(gu + r * 2 * di + di + c);
    Vec8<T> o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float gate = to_f32(g.v[e]);
        o.v[e] = from_f32<T>(gate * (1.0f / (1.0f + expf(-gate))) * to_f32(u.v[e]));
    }
    *(Vec8<T> *)(out + r * di + c) = o;
}

LCU_API int lcu_swiglu(void *out, const void *gate_up, int type, int n, int di, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (di <= 0) return LCU_BAD_ARGUMENT;
    dim3 block(256);
    // grid.y is limited to 65535 rows: larger batches go in slices
    for (int r0 = 0; r0 < n; r0 += 65535) {
        const int rows = (n - r0) < 65535 ? (n - r0) : 65535;
        dim3 grid((di + 255) / 256, rows);
        if (di % 8 == 0) {
            dim3 vgrid((di / 8 + 255) / 256, rows);
            if (type == LCU_F32)
                swiglu_vec8_kernel<float><<<vgrid, block, 0, stream>>>((float *)out + (size_t)r0 * di, (const float *)gate_up + (size_t)r0 * 2 * di, di);
            else if (type == LCU_BF16)
                swiglu_vec8_kernel<bf16_t><<<vgrid, block, 0, stream>>>((bf16_t *)out + (size_t)r0 * di, (const bf16_t *)gate_up + (size_t)r0 * 2 * di, di);
            else
                return LCU_BAD_ARGUMENT;
            continue;
        }
        if (type == LCU_F32)
            swiglu_kernel<float><<<grid, block, 0, stream>>>((float *)out + (size_t)r0 * di, (const float *)gate_up + (size_t)r0 * 2 * di, di);
        else if (type == LCU_BF16)
            swiglu_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t *)out + (size_t)r0 * di, (const bf16_t *)gate_up + (size_t)r0 * 2 * di, di);
        else
            return LCU_BAD_ARGUMENT;
    }
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- token feedback
// tokens[dst[i]] = sampled[src[i]]: the ids that the last step sampled become this step's
// inputs on the device, so the host need not wait for them before it launches
// (llama.cu/src/op/fast_embedding.cuh:1-15 does the same from its sampled pairs).
__global__ void feed_tokens_kernel(int *__restrict__ tokens, const int *__restrict__ sampled,
                                   const int *__restrict__ src, const int *__restrict__ dst, int n, int n_tokens,
                                   int n_sampled) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int s = src[i], d = dst[i];
    if (s >= 0 && s < n_sampled && d >= 0 && d < n_tokens) tokens[d] = sampled[s];
}

LCU_API int lcu_feed_tokens(int *tokens, int n_tokens, const int *sampled, int n_sampled, const int *src, const int *dst,
                            int n, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    feed_tokens_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(tokens, sampled, src, dst, n, n_tokens, n_sampled);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
