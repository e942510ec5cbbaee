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
            float ra, rb;
            rotate_pair(a, b, c, s, ra, rb);
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
                float xa, xb;
                rotate_pair(fa, fb, c, s, xa, xb);
                ra.v[e] = from_f32<T>(xa);
                rb.v[e] = from_f32<T>(xb);
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

// The same for many tokens: a block takes eight neighbouring tokens of the batch, so that the
// values of one dim, which lie along the tokens in a page, leave as one 16- or 32-byte store
// when the eight tokens stand in a row in one page (a prompt's portion that starts at a
// multiple of eight); otherwise element by element.
template <class T>
__global__ void __launch_bounds__(256)
rope_kv_store_half_tokens8_kernel(T *__restrict__ qkv, int row_stride, int n, const int *__restrict__ positions,
                                  const int *__restrict__ slots, const float *__restrict__ cos_t,
                                  const float *__restrict__ sin_t, int max_pos, T *__restrict__ cache, int nh, int nkvh,
                                  int dh, int page) {
    const int t0 = blockIdx.x * 8;
    const int nt = min(8, n - t0);
    const int half = dh / 2;
    const int per_head = half / 8;
    const int n_rot = (nh + nkvh) * per_head;               // per token
    const int n_val = nkvh * dh;                            // per group of eight tokens
    const int w = blockIdx.y * blockDim.x + threadIdx.x;
    if (w < 8 * n_rot) {
        const int e_t = w / n_rot, item = w % n_rot;
        if (e_t >= nt) return;
        const int t = t0 + e_t;
        T *row = qkv + (size_t)t * row_stride;
        const int pos = positions[t];
        const bool in_table = pos >= 0 && pos < max_pos;
        const int head = item / per_head, i0 = (item % per_head) * 8;
        T *x = row + (size_t)head * dh;
        const Row8<T> a = *(const Row8<T> *)(x + i0), b = *(const Row8<T> *)(x + half + i0);
        float c[8], sn[8];
        if (in_table) {
            const float4 *cp = (const float4 *)(cos_t + (size_t)pos * half + i0), *sp = (const float4 *)(sin_t + (size_t)pos * half + i0);
            const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
            c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
            sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) c[e] = sn[e] = __uint_as_float(0x7fc00000u);   // a position outside the table gives NaN
        }
        Row8<T> ra, rb;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float fa = to_f32(a.v[e]), fb = to_f32(b.v[e]);
            float xa, xb;
            rotate_pair(fa, fb, c[e], sn[e], xa, xb);
            ra.v[e] = from_f32<T>(xa);
            rb.v[e] = from_f32<T>(xb);
        }
        if (head < nh) {
            *(Row8<T> *)(x + i0) = ra;
            *(Row8<T> *)(x + half + i0) = rb;
        } else {
            const int slot = slots[t];
            if (slot >= 0) {
                T *pg = cache + (size_t)(slot / page) * kv_page_elems(nkvh, dh, page);
                const int kvh = head - nh, tok = slot % page;
                *(Row8<T> *)(pg + kv_key_offset(kvh, tok, i0, dh, page)) = ra;
                *(Row8<T> *)(pg + kv_key_offset(kvh, tok, half + i0, dh, page)) = rb;
            }
        }
        return;
    }
    const int v = w - 8 * n_rot;
    if (v >= n_val) return;
    const int kvh = v / dh, dim = v % dh;
    const T *src = qkv + (size_t)t0 * row_stride + (size_t)(nh + nkvh) * dh + (size_t)kvh * dh + dim;
    const int slot0 = slots[t0];
    bool row8 = nt == 8 && slot0 >= 0 && slot0 % 8 == 0;     // page sizes are multiples of 8: such a run stays in its page
#pragma unroll
    for (int e = 1; e < 8; ++e) row8 = row8 && (e >= nt || slots[t0 + e] == slot0 + e);
    if (row8) {
        Row8<T> val;
#pragma unroll
        for (int e = 0; e < 8; ++e) val.v[e] = src[(size_t)e * row_stride];
        T *pg = cache + (size_t)(slot0 / page) * kv_page_elems(nkvh, dh, page);
        *(Row8<T> *)(pg + kv_value_offset(nkvh, kvh, slot0 % page, dim, dh, page)) = val;
    } else {
        for (int e = 0; e < nt; ++e) {
            const int slot = slots[t0 + e];
            if (slot < 0) continue;
            T *pg = cache + (size_t)(slot / page) * kv_page_elems(nkvh, dh, page);
            pg[kv_value_offset(nkvh, kvh, slot % page, dim, dh, page)] = src[(size_t)e * row_stride];
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
        if (store_kv && n >= 64 && (size_t)cos_t % 16 == 0 && (size_t)sin_t % 16 == 0) {
            const int items8 = 8 * (nh + nkvh) * (dh / 16) + nkvh * dh;
            const dim3 g8((n + 7) / 8, (items8 + 255) / 256);
            if (type == LCU_F32)
                rope_kv_store_half_tokens8_kernel<float><<<g8, dim3(256), 0, stream>>>((float *)qkv, row_stride, n, positions, slots, cos_t, sin_t, max_pos, (float *)cache, nh, nkvh, dh, page);
            else
                rope_kv_store_half_tokens8_kernel<bf16_t><<<g8, dim3(256), 0, stream>>>((bf16_t *)qkv, row_stride, n, positions, slots, cos_t, sin_t, max_pos, (bf16_t *)cache, nh, nkvh, dh, page);
            LCU_LAUNCH_CHECK();
            return LCU_OK;
        }
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
