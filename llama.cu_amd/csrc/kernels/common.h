// Shared device helpers for the gfx950 kernels: element types, conversions,
// wave and block reductions.  A wave has 64 lanes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LCU_API extern "C" __attribute__((visibility("default")))

// Error codes returned by every entry point (0 = launched).
enum { LCU_OK = 0, LCU_BAD_ARGUMENT = -1, LCU_UNSUPPORTED = -2 };

// Element type codes shared with the Python side.
enum { LCU_F32 = 0, LCU_BF16 = 1 };

struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }

template <class T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
// round to nearest, ties to even; NaN stays NaN (the hardware's v_cvt_pk_bf16_f32)
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) {
    const __bf16 b = (__bf16)x;
    bf16_t r;
    r.bits = __builtin_bit_cast(uint16_t, b);
    return r;
}
// two at once, packed into 32 bits (lo in the low half)
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

constexpr int WAVE = 64;

// The rotation of one pair (a, b) by an angle with cosine c and sine s, rounded the same way in
// every kernel that rotates: one product rounded, the other fused into the sum, written out so
// that the compiler has no choice of its own.  A token's rotated values then do not depend on
// which kernel its batch was given to.
__device__ inline void rotate_pair(float a, float b, float c, float s, float &ra, float &rb) {
#pragma clang fp contract(off)
    const float bs = b * s, bc = b * c;
    ra = __builtin_fmaf(a, c, -bs);
    rb = __builtin_fmaf(a, s, bc);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds 16 floats of LDS.  Every
// thread gets the result.  The order of the additions depends on the block's size
// only.
__device__ __forceinline__ float block_sum(float v, float *scratch) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nwaves; ++i) t += scratch[i];
    return t;
}

// A workgroup barrier that waits for this wave's LDS accesses only.  __syncthreads() also
// waits until every global load of the wave has come back, which empties a software
// pipeline that keeps loads of later steps in flight across the barrier.  Use it where the
// waves exchange data through LDS only.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

#define LCU_LAUNCH_CHECK()                                   \
    do {                                                     \
        hipError_t e_ = hipGetLastError();                   \
        if (e_ != hipSuccess) return (int)e_;                \
    } while (0)
