// An entry point of the attention library that allocates nothing.
//
// It has no counterpart in the reference (YdrMaster/llama.cu), whose attention operator takes its
// workspace from the caller's arena.  It is for callers that cannot allocate: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  lcu_attention_decode_bf16 cuts a
// request's keys into `n_splits` parts and needs device memory for the parts' partial results
// (part_o, part_ml), which its caller brings.  This variant takes that memory from a buffer of
// fixed size that lives in the library's own device image, so the caller passes inputs and outputs
// only and no call on its path allocates or frees (no hipMalloc, no hipFree, no library routine
// that allocates).
//
//   * The buffer holds LCU_ATTENTION_STATIC_SCRATCH_BYTES (16 MiB) on every GPU that the library
//     runs on, until the process ends.  A call needs n_req * heads * n_splits * (head_dim + 2) * 4
//     bytes of it (nothing when n_splits == 1); a call that needs more is refused with
//     LCU_SCRATCH_EXCEEDED (-3) and launches nothing.
//   * Every call on a GPU uses that GPU's one buffer: calls that may run at the same time on one
//     GPU (different streams, different threads) race on it.  Calls on one stream are in order
//     and safe.  Nothing in the buffer has to start at zero: the decode kernel writes every slot
//     that the merge kernel reads, so the last call's contents do no harm.
//   * The buffer's address is looked up once per device (hipGetSymbolAddress, with that device
//     current) by lcu_attention_static_init or by the entry point's first call on the device; call
//     lcu_attention_static_init beforehand where even that look-up is unwelcome (before a capture).
//
// All other arguments are those of lcu_attention_decode_bf16, and they are checked as there (and first: a call
// with sizes that no kernel takes gets LCU_BAD_ARGUMENT or LCU_UNSUPPORTED, not LCU_SCRATCH_EXCEEDED).
#pragma once
#include <hip/hip_runtime.h>

#define LCU_ATTENTION_STATIC_SCRATCH_BYTES (16u << 20)
#define LCU_SCRATCH_EXCEEDED (-3)
#define LCU_RUNTIME_ERROR (-4)      // the HIP runtime refused a call that is no launch (the buffer's address, the device)

extern "C" {
// Looks the buffer's address up for the current device; 0, LCU_UNSUPPORTED (-2: a device number of 64 or more)
// or LCU_RUNTIME_ERROR.
int lcu_attention_static_init(void);
// The size of the buffer in bytes.
long long lcu_attention_static_scratch_bytes(void);
// The bytes of the buffer that a call with these sizes uses.
long long lcu_attention_static_scratch_needed(int n_req, int nh, int dh, int n_splits);
int lcu_attention_decode_bf16_static(const void *q, int q_stride, void *out, int out_stride, const void *cache,
                                     const int *block_table, int max_pages, const int *q_start, const int *ctx_len,
                                     const int *req_list, int n_req, int nh, int nkvh, int dh, int page, float scale,
                                     int window, int n_splits, hipStream_t stream);
}
