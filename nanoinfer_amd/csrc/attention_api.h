// C interface of the token-at-a-time attention library (attention.hip, one library per head size).
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Attention of T_tokens query tokens over the paged cache.  q: [T, q_stride] with the H rotated
// query heads first; pools [pages, KVH, page_size, HEAD_DIM]; block_table int32 [sequences,
// table_stride]; out [T, H*HEAD_DIM].  With nsplit > 1 the key range of every token is cut into
// nsplit runs whose partial results go through the caller's workspace: part_o float
// [T, H, nsplit, HEAD_DIM], part_ml float [T, H, nsplit, 2].  dtype 0: float32, 1: bfloat16.
// Returns 0 or a HIP error code; -1 / -2 for arguments it refuses.
int ni_token_attention(const void* q, int q_stride, const void* kpool, const void* vpool, const void* block_table,
                       int table_stride, const void* seq_of_token, const void* positions, void* out, void* part_o,
                       void* part_ml, int T_tokens, int H, int KVH, int page_size, int window, float scale, int nsplit,
                       int dtype, hipStream_t stream);

// The same attention for callers that cannot allocate device memory and so cannot bring a
// workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// It has no counterpart in the reference (whose attention allocates its temporaries with
// cudaMallocAsync on every call).  The partial results of the key runs live in an array that the
// library itself holds in device memory, ni_token_attention_static_floats() floats (4 MiB) on
// every GPU the library runs on, until the process ends.  The call allocates nothing, frees
// nothing and calls no routine that does.  It needs T_tokens * H * nsplit * (HEAD_DIM + 2) floats:
// more than the array holds is refused with -3 and nothing is launched.  Nothing in the array has
// to start at zero (every run writes its place before the merge reads it), so nothing is cleared.
// All calls on one GPU share that GPU's array: two calls whose kernels overlap in time (on
// different streams, or from different threads) race on it; calls on one stream do not.
int ni_token_attention_static(const void* q, int q_stride, const void* kpool, const void* vpool,
                              const void* block_table, int table_stride, const void* seq_of_token,
                              const void* positions, void* out, int T_tokens, int H, int KVH, int page_size,
                              int window, float scale, int nsplit, int dtype, hipStream_t stream);

// Capacity of the library's own array, in floats.
long ni_token_attention_static_floats(void);

#ifdef __cplusplus
}
#endif
