// Entry points of the library that callers other than this package's own Python
// wrappers are meant to use directly.  C ABI, raw device pointers, a HIP stream.
// Every function returns 0 on success; on refusal a negative code, with the reason
// readable through mi_last_error().
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Size of the library's own scratch array that mi_attn_generic_static uses (bytes).
#define MI_ATTN_STATIC_SCRATCH_BYTES (8u << 20)

// Paged causal attention with the keys cut into `num_splits` ranges, like
// mi_attn_generic, for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
// counterpart in the reference engine, whose attention always takes its workspace
// from the framework's allocator.
//
// The partial results of the key ranges (num_tokens * q_heads * num_splits *
// (head_dim + 2) floats) lie in an array inside the library instead of in buffers
// the caller brings: MI_ATTN_STATIC_SCRATCH_BYTES per GPU, held from the first call
// on that GPU until the process ends.  A call whose partial results would not fit is
// refused with an error and nothing is launched.  The call itself allocates and frees
// nothing.  All calls on one GPU share that GPU's array: calls that may overlap on one
// GPU (different streams, several threads) race on it and must be serialized by the
// caller; calls on one stream are ordered.  Nothing in the array has to be cleared
// between calls: every call writes all the entries it reads.
//
// Arguments, layouts and results are those of mi_attn_generic (dtype 0 = float32,
// 1 = bfloat16; `slopes` may be null); the output is bit-identical to it for the same
// `num_splits`.
int mi_attn_generic_static(int dtype, const void* q, int64_t q_row_stride, const void* k_pages,
                           const void* v_pages, const int* block_table, int max_blocks,
                           const int* token_request, const int* positions, void* out,
                           int64_t out_row_stride, int num_tokens, int q_heads, int kv_heads,
                           int head_dim, int page_size, int num_pages, float scale, int window,
                           int num_splits, const float* slopes, hipStream_t stream);

#ifdef __cplusplus
}
#endif
