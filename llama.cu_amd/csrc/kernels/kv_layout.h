// The layout of one page of the key/value cache, shared by the kernel that writes
// it and the kernels that read it.
//
// One layer's cache is [num_pages][2][kv_heads * head_dim * page_size] elements: in a
// page first all keys, then all values.
//   keys:   [kv_head][head_dim / 8][token in page][8]   eight neighbouring dims of one
//           token are contiguous and tokens follow each other: lanes that hold
//           neighbouring tokens read neighbouring 16 (bf16) or 32 (f32) bytes.
//   values: [kv_head][dim][token in page]               the tokens of one dim are
//           contiguous: a lane that owns a dim reads a run of tokens.
// head_dim is a multiple of 8 (the engine asks for 16), page_size a multiple of 8.
#pragma once
#include <stddef.h>

__host__ __device__ inline size_t kv_page_elems(int kv_heads, int head_dim, int page) {
    return (size_t)2 * kv_heads * head_dim * page;
}
__host__ __device__ inline size_t kv_key_offset(int kv_head, int tok, int dim, int head_dim, int page) {
    return (((size_t)kv_head * (head_dim / 8) + dim / 8) * page + tok) * 8 + (dim & 7);
}
__host__ __device__ inline size_t kv_value_offset(int kv_heads, int kv_head, int tok, int dim, int head_dim, int page) {
    return (size_t)kv_heads * head_dim * page + ((size_t)kv_head * head_dim + dim) * page + tok;
}
