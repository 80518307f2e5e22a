// Entry points that allocate nothing.
//
// kappai has no counterpart of these: its backends size and allocate their workspaces when a
// session is created.  They are for callers that cannot allocate device memory at the time of
// the call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// Such an entry point is a variant of an existing one whose workspace argument is replaced by
// a file-scope device array of a fixed, stated size inside the library; the caller passes only
// inputs and outputs, and nothing in the call allocates or frees (no hipMalloc, no hipFree, no
// allocating library routine).
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Floats of the device array that kappai_attn_decode_static keeps its partial results in
// (4 MiB; every GPU that the library runs on holds one such array until the process ends).
#define KAPPAI_ATTN_STATIC_SCRATCH_FLOATS (1 << 20)

// The number of floats above, for callers that size their work at run time.
int kappai_attn_decode_static_capacity(void);

// Looks up the address of the current device's copy of the array (hipGetSymbolAddress) and keeps
// it; returns 0 or the hipError_t of the lookup.  kappai_attn_decode_static does this by itself
// at its first call on a device; a caller that captures graphs calls it once before the capture.
int kappai_attn_decode_static_init(void);

// kappai_attn_decode (split-key decode attention over the paged cache, then the merge of the
// splits) without the two workspace arguments: the partial results
//     part_o  [T, H, n_splits, HEAD_DIM] float   and   part_ml [T, H, n_splits, 2] float
// live in the library's own device array.  Same inputs, same output, same kernels, bit for bit.
// (n_splits is the most splits a row may have and keys_per_split the fewest keys of a split, as
// for kappai_attn_decode: the kernels settle on the keys per split from the rows' lengths, and
// the splits past a row's keys are neither written nor read.)
// Returns hipErrorInvalidValue, with a message that kappai_attn_decode_static_error() returns,
// when T * H * n_splits * (HEAD_DIM + 2) exceeds KAPPAI_ATTN_STATIC_SCRATCH_FLOATS or an
// argument is one that kappai_attn_decode refuses.
// Every call on a GPU uses that GPU's one array, which keeps the last call's contents: the
// kernels write every partial result they later read, so nothing has to be cleared, but two
// calls that overlap on one GPU (two streams, two threads) race on it.  Calls on one stream,
// or on streams that are ordered by events, are safe.
int kappai_attn_decode_static(const void* q, int q_stride, const void* k_pool, const void* vt_pool,
                              void* out, int out_stride, const int* row_pos, const int* row_seg,
                              const int* block_tables, int max_blocks, int T, int H, int G, int ps,
                              int window, float scale, int keys_per_split, int n_splits,
                              hipStream_t stream);

// The message of this thread's last refused call ("" if none).
const char* kappai_attn_decode_static_error(void);

#ifdef __cplusplus
}
#endif
