// A counter-based generator of standard normal numbers, one source for the host and the GPU.
//
// Element i of a stream with the 64-bit key `key` is
//     z  = mix64(key + (i + 1) * 0x9E3779B97F4A7C15)          (the finalizer of splitmix64)
//     u1 = (high 32 bits of z + 0.5) / 2^32,  u2 = (low 32 bits of z + 0.5) / 2^32     in (0, 1)
//     x  = sqrt(-2 ln u1) * cos(2 pi u2)                       (Box-Muller)
// in 64-bit arithmetic that uses only operations which IEEE 754 rounds exactly (+, -, *, /, sqrt,
// no fused multiply-add) in one fixed order, with the logarithm and the cosine as polynomials
// written out here: the host's C++ compiler and the GPU's give the same bits.  The logarithm:
// u1 = m 2^e with m in [sqrt(1/2), sqrt(2)), ln m = 2 atanh(s), s = (m - 1) / (m + 1), |s| < 0.172,
// the series up to s^13 (error below 2e-11).  The cosine: 4 u2 = q + f, x = f pi / 2, the Taylor
// series of cos x and sin x up to x^16 and x^17 (error below 1e-12), the quadrant q picks and signs.
// The value is then rounded to 32-bit once.  A stream does not depend on how many elements are
// made, by whom, or in what order.
#pragma once
#include <stdint.h>
#include <math.h>
#include <string.h>

#ifdef __HIPCC__
#define LCU_HD __host__ __device__ inline
#else
#define LCU_HD inline
#endif

LCU_HD uint64_t lcu_mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27;
    z *= 0x94D049BB133111EBull;
    z ^= z >> 31;
    return z;
}

LCU_HD double lcu_standard_normal(uint64_t key, uint64_t index) {
#ifdef __clang__
#pragma clang fp contract(off)
#endif
    const uint64_t z = lcu_mix64(key + (index + 1) * 0x9E3779B97F4A7C15ull);
    const double u1 = ((double)(uint32_t)(z >> 32) + 0.5) * 2.3283064365386963e-10;        // 2^-32: exact
    const double u2 = ((double)(uint32_t)(z & 0xffffffffu) + 0.5) * 2.3283064365386963e-10;
    // ---- ln u1: exponent and mantissa by their bits (u1 is a normal number)
    uint64_t bits;
    memcpy(&bits, &u1, 8);
    int e = (int)((bits >> 52) & 0x7ff) - 1022;                        // u1 = m 2^e, m in [1/2, 1)
    bits = (bits & 0x000fffffffffffffull) | 0x3fe0000000000000ull;
    double m;
    memcpy(&m, &bits, 8);
    if (m < 0.70710678118654757) { m = m * 2.0; e -= 1; }              // m in [sqrt(1/2), sqrt(2))
    const double s = (m - 1.0) / (m + 1.0);
    const double s2 = s * s;
    double p = 0.07692307692307693;
    p = p * s2 + 0.09090909090909091;
    p = p * s2 + 0.1111111111111111;
    p = p * s2 + 0.14285714285714285;
    p = p * s2 + 0.2;
    p = p * s2 + 0.3333333333333333;
    p = p * s2 + 1.0;
    const double ln_u1 = (double)e * 0.69314718055994529 + 2.0 * (s * p);
    const double r = sqrt(-2.0 * ln_u1);
    // ---- cos(2 pi u2)
    const double t = u2 * 4.0;                                         // exact
    const int q = (int)t;                                              // 0 .. 3
    const double x = (t - (double)q) * 1.5707963267948966;             // in [0, pi / 2)
    const double x2 = x * x;
    double c = 4.779477332387385e-14;
    c = c * x2 + -1.1470745597729725e-11;
    c = c * x2 + 2.08767569878681e-09;
    c = c * x2 + -2.755731922398589e-07;
    c = c * x2 + 2.48015873015873e-05;
    c = c * x2 + -0.001388888888888889;
    c = c * x2 + 0.041666666666666664;
    c = c * x2 + -0.5;
    c = c * x2 + 1.0;
    double sn = 2.8114572543455206e-15;
    sn = sn * x2 + -7.647163731819816e-13;
    sn = sn * x2 + 1.6059043836821613e-10;
    sn = sn * x2 + -2.505210838544172e-08;
    sn = sn * x2 + 2.7557319223985893e-06;
    sn = sn * x2 + -0.0001984126984126984;
    sn = sn * x2 + 0.008333333333333333;
    sn = sn * x2 + -0.16666666666666666;
    sn = sn * x2 + 1.0;
    sn = sn * x;
    const double trig = q == 0 ? c : (q == 1 ? -sn : (q == 2 ? -c : sn));
    return r * trig;
}

// One weight: 32-bit value = (32-bit normal) * std + shift, the product rounded, then the sum rounded.
LCU_HD float lcu_random_weight(uint64_t key, uint64_t index, float std, float shift) {
#ifdef __clang__
#pragma clang fp contract(off)
#endif
    const float n = (float)lcu_standard_normal(key, index);
    const float scaled = n * std;
    return scaled + shift;
}

// 32-bit to bfloat16, round to nearest, ties to even (the values here are finite).
LCU_HD uint16_t lcu_bf16_bits(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
