// C[M, N] (+)= A[M, K] * W[N, K]^T with 32-bit accumulation, for every size and for
// 32-bit and bfloat16 operands in any mix.  This is the true 32-bit matrix product
// of the engine (plain multiply-adds on 32-bit values, no reduced-precision matrix
// mode) and the fallback of the bfloat16 path for shapes its faster kernels refuse.
//
// A 64x64 tile per block of 256 threads, 4x4 outputs per thread, K in steps of 16
// through LDS.  Every output adds its K products in the order k = 0, 1, 2, ...: a
// row's result does not depend on M or on the other rows of the batch.
#include "common.h"

constexpr int BM = 64, BN = 64, BK = 16;

template <class TA, class TW, class TO, bool ACCUMULATE>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const TA *__restrict__ A, int lda, const TW *__restrict__ W, int ldw, TO *__restrict__ C, int ldc,
               int M, int N, int K) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256;
            const int row = idx / BK, kk = idx % BK;
            const int gm = m0 + row, gn = n0 + row, gk = k0 + kk;
            As[kk][row] = (gm < M && gk < K) ? to_f32(A[(size_t)gm * lda + gk]) : 0.f;
            Ws[kk][row] = (gn < N && gk < K) ? to_f32(W[(size_t)gn * ldw + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn >= N) continue;
            TO *c = C + (size_t)gm * ldc + gn;
            float v = acc[i][j];
            if (ACCUMULATE) v += to_f32(*c);
            *c = from_f32<TO>(v);
        }
    }
}

template <class TA, class TW, class TO>
static int launch(const void *A, int lda, const void *W, int ldw, void *C, int ldc, int M, int N, int K,
                  int accumulate, hipStream_t stream) {
    dim3 block(256);
    // grid.y is limited to 65535 tiles: larger M goes in slices
    const int max_rows = 65535 * BM;
    for (int r0 = 0; r0 < M; r0 += max_rows) {
        const int rows = (M - r0) < max_rows ? (M - r0) : max_rows;
        dim3 grid((N + BN - 1) / BN, (rows + BM - 1) / BM);
        const TA *a = (const TA *)A + (size_t)r0 * lda;
        TO *c = (TO *)C + (size_t)r0 * ldc;
        if (accumulate)
            gemm_nt_kernel<TA, TW, TO, true><<<grid, block, 0, stream>>>(a, lda, (const TW *)W, ldw, c, ldc, rows, N, K);
        else
            gemm_nt_kernel<TA, TW, TO, false><<<grid, block, 0, stream>>>(a, lda, (const TW *)W, ldw, c, ldc, rows, N, K);
    }
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// A: [M, K] rows lda apart, W: [N, K] rows ldw apart, C: [M, N] rows ldc apart.
// accumulate: C = C + A W^T (the sum in 32-bit, one rounding).
LCU_API int lcu_gemm_nt(const void *A, int a_type, int lda, const void *W, int w_type, int ldw, void *C, int c_type,
                        int ldc, int M, int N, int K, int accumulate, hipStream_t stream) {
    if (M <= 0 || N <= 0) return LCU_OK;
    if (K <= 0 || lda < K || ldw < K || ldc < N) return LCU_BAD_ARGUMENT;
    const int key = a_type * 4 + w_type * 2 + c_type;
    switch (key) {
    case 0: return launch<float, float, float>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 1: return launch<float, float, bf16_t>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 2: return launch<float, bf16_t, float>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 3: return launch<float, bf16_t, bf16_t>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 4: return launch<bf16_t, float, float>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 5: return launch<bf16_t, float, bf16_t>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 6: return launch<bf16_t, bf16_t, float>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    case 7: return launch<bf16_t, bf16_t, bf16_t>(A, lda, W, ldw, C, ldc, M, N, K, accumulate, stream);
    }
    return LCU_BAD_ARGUMENT;
}
