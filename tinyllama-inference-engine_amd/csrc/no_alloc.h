// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
// code that runs under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// The library's other entry points leave scratch memory (the partial results of attention's key
// parts) to their caller, who brings it as arguments; Python's face allocates it through torch.
#pragma once

#include <stddef.h>

// The size of the scratch array that every GPU the library runs on holds until the process ends.
#define TLIE_NO_ALLOC_SCRATCH_BYTES (8u << 20)

#ifdef __cplusplus
extern "C" {
#endif

// tlie_attention_mfma (paged causal grouped-query attention, bfloat16: attention_mfma.hip) with the
// partial results of the `nsplit` key parts kept in a file-scope device array of
// TLIE_NO_ALLOC_SCRATCH_BYTES instead of buffers of the caller's: all other arguments, their
// meaning, the kernels and the results (bit for bit) are those of tlie_attention_mfma.
//
// It calls no hipMalloc, hipFree or other allocating routine.  Returns 0 when launched; -1 for
// sizes or types the kernel does not take; -2 when a launch or the look-up of the array's address
// failed; -4 when tokens * nq * nsplit * (d + 2) floats (the rows of d rounded up to 256 bytes in
// all) do not fit the array: such a step needs the entry point that takes buffers.
//
// Every call on a GPU uses that GPU's one array, which keeps the last call's contents; a call
// writes every entry it reads, so nothing has to be cleared.  Two calls that overlap in time on one
// GPU (on two streams, say) race for the array: a caller runs them one after the other.
int tlie_attention_mfma_no_alloc(const void* q, const void* cache, const int* block_table, int max_blocks,
                                 const void* tiles, int num_tiles, int col_tiles, const int* positions, void* out,
                                 int nsplit, int split_len, int tokens, int nq, int nkv, int d, int page_size,
                                 int window, float scale, int waves, int shared, void* stream);

#ifdef __cplusplus
}
#endif
