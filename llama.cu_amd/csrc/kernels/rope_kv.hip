// Rotary position encoding of the queries and keys of one step, fused with the write
// of the step's keys and values into their pages.
//
// The rotation of one pair (a, b) by the angle of its token's position:
//   (a, b) -> (a*cos - b*sin, a*sin + b*cos)
// computed in 32-bit from 32-bit tables [max_pos, rot_dim/2], one rounding at the
// store.  pairing 0: the pair is (x[i], x[i + rot_dim/2]); pairing 1: (x[2i], x[2i+1]).
// Dims at and above rot_dim are not rotated.  A null table means no rotation at all.
#include "common.h"
#include "kv_layout.h"

// One block per (token, head): query heads are rotated in place, key heads are rotated into
// the cache, value heads are copied into the cache.
template <class T>
__global__ void rope_kv_store_kernel(T *__restrict__ qkv, int row_stride, const int *__restrict__ positions,
                                     const int *__restrict__ slots, const float *__restrict__ cos_t,
                                     const float *__restrict__ sin_t, int max_pos, T *__restrict__ cache,
                                     int nh, int nkvh, int dh, int rot_dim, int pairing, int page,
                                     int store_kv) {
    const int t = blockIdx.x, head = blockIdx.y;
    T *x = qkv + (size_t)t * row_stride + (size_t)head * dh;
    const int pos = positions[t];
    const int half = rot_dim / 2;
    const bool in_table = pos >= 0 && pos < max_pos;
    const bool rotate = cos_t != nullptr && in_table;
    // a position outside the table (the host checks before) gives NaN, not a wrong value
    const bool poison = cos_t != nullptr && !in_table;
    const int slot = store_kv ? slots[t] : -1;
    T *pg = nullptr;
    int tok = 0;
    if (slot >= 0) {
        pg = cache + (size_t)(slot / page) * kv_page_elems(nkvh, dh, page);
        tok = slot % page;
    }
    if (head >= nh + nkvh) {                    // a value head: copied as it is
        if (!pg) return;
        const int kvh = head - nh - nkvh;
        for (int c = threadIdx.x; c < dh; c += blockDim.x) pg[kv_value_offset(nkvh, kvh, tok, c, dh, page)] = x[c];
        return;
    }
    const bool is_key = head >= nh;
    if (is_key && !pg) return;
    if (!is_key && !rotate && !poison) return;  // a query head that is not rotated stays as it is
    for (int i = threadIdx.x; i < dh / 2; i += blockDim.x) {
        int ia, ib;
        const bool rot = rotate && i < half;
        if (i < half) {                // a rotated pair
            if (pairing == 0) { ia = i; ib = i + half; } else { ia = 2 * i; ib = 2 * i + 1; }
        } else {                       // dims at and above rot_dim pass through, two at a time
            ia = rot_dim + 2 * (i - half); ib = ia + 1;
        }
        float a = to_f32(x[ia]), b = to_f32(x[ib]);
        if (rot) {
            const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
            const float ra = a * c - b * s, rb = a * s + b * c;
            a = ra; b = rb;
        }
        if (poison && i < half) a = b = __uint_as_float(0x7fc00000u);
        const T va = from_f32<T>(a), vb = from_f32<T>(b);
        if (!is_key) {
            if (rot || poison) { x[ia] = va; x[ib] = vb; }
        } else {
            const int kvh = head - nh;
            pg[kv_key_offset(kvh, tok, ia, dh, page)] = va;
            pg[kv_key_offset(kvh, tok, ib, dh, page)] = vb;
        }
    }
}

// The common case in one pass with wide accesses: the whole head is rotated, the pairs are
// (i, i + dh/2), dh a multiple of 16.  A thread takes 8 neighbouring pairs of one head of
// one token (two 8-element loads), or 8 elements of a value head.
template <class T> struct alignas(8 * sizeof(T)) Row8 { T v[8]; };

template <class T>
__global__ void __launch_bounds__(256)
rope_kv_store_half_kernel(T *__restrict__ qkv, int row_stride, const int *__restrict__ positions,
                          const int *__restrict__ slots, const float *__restrict__ cos_t,
                          const float *__restrict__ sin_t, int max_pos, T *__restrict__ cache, int nh, int nkvh, int dh,
                          int page, int store_kv) {
    const int t = blockIdx.x;
    T *row = qkv + (size_t)t * row_stride;
    const int pos = positions[t];
    const int half = dh / 2;
    const bool in_table = pos >= 0 && pos < max_pos;
    const int slot = store_kv ? slots[t] : -1;
    T *pg = nullptr;
    int tok = 0;
    if (slot >= 0) {
        pg = cache + (size_t)(slot / page) * kv_page_elems(nkvh, dh, page);
        tok = slot % page;
    }
    const int per_head = half / 8;                        // work items of a rotated head
    const int n_rot = (nh + (store_kv ? nkvh : 0)) * per_head;
    const int n_val = store_kv ? nkvh * dh / 8 : 0;
    const int w = blockIdx.y * blockDim.x + threadIdx.x;
    if (w >= n_rot + n_val) return;
    {
        if (w < n_rot) {
            const int head = w / per_head, i0 = (w % per_head) * 8;
            T *x = row + (size_t)head * dh;
            const Row8<T> a = *(const Row8<T> *)(x + i0), b = *(const Row8<T> *)(x + half + i0);
            Row8<T> ra, rb;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float fa = to_f32(a.v[e]), fb = to_f32(b.v[e]);
                float c = __uint_as_float(0x7fc00000u), s = c;      // a position outside the table gives NaN
                if (in_table) { c = cos_t[(size_t)pos * half + i0 + e]; s = sin_t[(size_t)pos * half + i0 + e]; }
                ra.v[e] = from_f32<T>(fa * c - fb * s);
                rb.v[e] = from_f32<T>(fa * s + fb * c);
            }
            if (head < nh) {
                *(Row8<T> *)(x + i0) = ra;
                *(Row8<T> *)(x + half + i0) = rb;
            } else if (pg) {
                const int kvh = head - nh;
                *(Row8<T> *)(pg + kv_key_offset(kvh, tok, i0, dh, page)) = ra;            // 8 dims of one token lie together
                *(Row8<T> *)(pg + kv_key_offset(kvh, tok, half + i0, dh, page)) = rb;
            }
        } else if (pg) {
            const int v = w - n_rot, kvh = v / (dh / 8), c0 = (v % (dh / 8)) * 8;
            const Row8<T> val = *(const Row8<T> *)(row + (size_t)(nh + nkvh) * dh + (size_t)kvh * dh + c0);
#pragma unroll
            for (int e = 0; e < 8; ++e) pg[kv_value_offset(nkvh, kvh, tok, c0 + e, dh, page)] = val.v[e];
        }
    }
}

// qkv: [n, row_stride] with a token's q heads, then k heads, then v heads (k and v only
// when store_kv).  cache: this layer's pages.  slots[t] = page * page_size + place in
// the page, or -1 to store nothing for token t.
LCU_API int lcu_rope_kv_store(void *qkv, int type, int n, int row_stride, const int *positions, const int *slots,
                              const float *cos_t, const float *sin_t, int max_pos, void *cache, int nh, int nkvh,
                              int dh, int rot_dim, int pairing, int page, int store_kv, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (dh <= 0 || dh % 8 || rot_dim % 2 || rot_dim > dh || rot_dim < 0 || page <= 0 || page % 8 || nh <= 0 ||
        nkvh < 0 || (pairing != 0 && pairing != 1))
        return LCU_BAD_ARGUMENT;
    if (store_kv && (!cache || !slots || nkvh <= 0)) return LCU_BAD_ARGUMENT;
    if (row_stride < (store_kv ? (nh + 2 * nkvh) : nh) * dh) return LCU_BAD_ARGUMENT;
    if (nh + 2 * nkvh > 65535) return LCU_BAD_ARGUMENT;
    const int elem = type == LCU_F32 ? 4 : 2;
    if (cos_t && pairing == 0 && rot_dim == dh && dh % 16 == 0 && (row_stride * elem) % (8 * elem) == 0 &&
        ((size_t)qkv % (8 * elem)) == 0 && (type == LCU_F32 || type == LCU_BF16)) {
        const int items = (nh + (store_kv ? nkvh : 0)) * (dh / 16) + (store_kv ? nkvh * dh / 8 : 0);
        const dim3 hgrid(n, (items + 255) / 256);
        if (type == LCU_F32)
            rope_kv_store_half_kernel<float><<<hgrid, dim3(256), 0, stream>>>((float *)qkv, row_stride, positions, slots, cos_t, sin_t, max_pos, (float *)cache, nh, nkvh, dh, page, store_kv);
        else
            rope_kv_store_half_kernel<bf16_t><<<hgrid, dim3(256), 0, stream>>>((bf16_t *)qkv, row_stride, positions, slots, cos_t, sin_t, max_pos, (bf16_t *)cache, nh, nkvh, dh, page, store_kv);
        LCU_LAUNCH_CHECK();
        return LCU_OK;
    }
    dim3 grid(n, store_kv ? nh + 2 * nkvh : nh), block(dh / 2 >= 64 ? 64 : 32);
    if (type == LCU_F32)
        rope_kv_store_kernel<float><<<grid, block, 0, stream>>>((float *)qkv, row_stride, positions, slots, cos_t, sin_t, max_pos, (float *)cache, nh, nkvh, dh, rot_dim, pairing, page, store_kv);
    else if (type == LCU_BF16)
        rope_kv_store_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t *)qkv, row_stride, positions, slots, cos_t, sin_t, max_pos, (bf16_t *)cache, nh, nkvh, dh, rot_dim, pairing, page, store_kv);
    else
        return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
