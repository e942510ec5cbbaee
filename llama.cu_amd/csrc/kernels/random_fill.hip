// Random weights made in place on the GPU: out[i] = normal(key, first + i) * std + shift, with the
// counter-based generator of csrc/shared/random_normal.h, which the host library compiles too, so
// that a model made on the GPU from a seed is bit for bit the model that the host writes to a
// folder from the same seed.  (The reference has no random-weights mode.)  The arithmetic is 64-bit
// and exactly rounded; the kernel runs once per tensor and is bound by that arithmetic, not by memory.
#include "common.h"
#include "../shared/random_normal.h"

template <class T>
__global__ void __launch_bounds__(256)
random_fill_kernel(T *__restrict__ out, long long n, unsigned long long key, long long first, float std, float shift) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float w = lcu_random_weight(key, (uint64_t)(first + i), std, shift);
        if constexpr (sizeof(T) == 4) {
            out[i] = w;
        } else {
            bf16_t b;
            b.bits = lcu_bf16_bits(w);
            out[i] = b;
        }
    }
}

// out: n elements of float32 (type LCU_F32) or bfloat16 (LCU_BF16).
LCU_API int lcu_random_fill(void *out, int type, long long n, unsigned long long key, long long first, float std, float shift,
                            hipStream_t stream) {
    if (n == 0) return LCU_OK;
    if (n < 0 || first < 0 || !out) return LCU_BAD_ARGUMENT;
    const long long blocks = (n + 255) / 256;
    const dim3 grid((unsigned)(blocks < 256 * 64 ? blocks : 256 * 64)), block(256);
    if (type == LCU_F32) random_fill_kernel<float><<<grid, block, 0, stream>>>((float *)out, n, key, first, std, shift);
    else if (type == LCU_BF16) random_fill_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t *)out, n, key, first, std, shift);
    else return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
