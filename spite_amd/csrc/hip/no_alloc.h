// Entry points of the kernel library that allocate nothing.
//
// No counterpart in the reference: they are for callers that cannot allocate device memory
// around a kernel call (code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc).  Such a caller passes inputs and outputs only; the scratch memory that
// the ordinary entry point takes as a workspace argument lives in a file-scope device array
// inside the library.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

// Floats of the library's own scratch array (16 MiB; each GPU that the library runs on holds
// it until the process ends).
#define SPITE_ATTN_DECODE_STATIC_FLOATS (4u << 20)

// spite_attn_decode with the splits' partial results kept in the library's scratch array
// instead of a workspace of the caller's: same kernels, same arguments otherwise, same result
// bit for bit.  Calls no hipMalloc, hipFree or allocating library routine.  A call whose
// partial results, T * H * n_splits * (hd + 2) floats, exceed
// SPITE_ATTN_DECODE_STATIC_FLOATS is refused with an error; with n_splits == 1 no scratch is
// used.  Every record of the scratch that the combining kernel reads is written by the same
// call before, so nothing has to be cleared; all calls on one GPU share that GPU's array, so
// calls that overlap on one GPU (different streams, different threads) race.
int spite_attn_decode_static(const void* q, const void* k_pages, const void* v_pages, void* out,
                             const int* positions, const int* seq_of_token, const int* block_table,
                             int max_blocks, int T, int H, int G, int hd, int page_size, int vis, int span,
                             float scale, int n_splits, hipStream_t st);

#ifdef __cplusplus
}
#endif
