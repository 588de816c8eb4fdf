// The one entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference (pekkah/SharpInference hands every kernel a buffer from
// its own pool).  It exists for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Largest workspace the entry point can stand in for, in floats (32 MiB).  Every GPU the library
// runs on holds one array of this size from the load of the library to the end of the process.
#define SHARPI_NOALLOC_SCRATCH_FLOATS (8u * 1024u * 1024u)

// sharpi_attention_decode without its two workspace arguments: the partial results of the
// key runs (n_list * nh * max_splits * (hd + 2) floats) live in a file-scope device array
// instead.  Same kernels, same results, same argument checks; additionally returns 1001 when the
// partial results would not fit SHARPI_NOALLOC_SCRATCH_FLOATS.  Calls no hipMalloc / hipFree and
// no allocating library routine; the caller passes inputs and the output as before.
//
// max_splits bounds the 256-key runs of a token: a token at position p whose first visible key is
// s needs ((p >> 4) - (s >> 4)) / 16 + 1 of them, and ((context - 1) >> 4) / 16 + 1 covers every
// token of a context whatever its window; a token that needs more than max_splits gets a row of
// NaN in `out` (never attention over fewer keys than it sees).
//
// The first call on a device looks up that device's copy of the array (hipGetSymbolAddress):
// make it outside a graph capture.  All calls on one GPU share that GPU's array, which keeps
// the last call's contents; nothing in it has to start at zero (every run that the merge reads
// is written by the call itself).  Two calls that overlap on one GPU (other streams, other
// threads) race on the array: order them.
__attribute__((visibility("default"))) int sharpi_attention_decode_noalloc(
    const void* q, const void* k_cache, const void* v_cache, const int* block_table, const int* entry_of_token,
    const int* positions, const int* token_list, void* out, int window_kind, int window, float scale, int n_list,
    int nh, int nkv, int hd, int page_size, int max_blocks, int num_pages, int max_splits, hipStream_t stream);

#ifdef __cplusplus
}
#endif
