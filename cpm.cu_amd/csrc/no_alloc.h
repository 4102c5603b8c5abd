// An entry point that allocates nothing.
//
// It has no counterpart in the reference engine.  It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Such a caller cannot
// bring the workspace that cpmcu_attention_mfma needs for the shares of a split-KV attention, so this
// variant keeps the shares in an array of the library's own (a file-scope __device__ array in
// attention.hip; every GPU the library runs on holds its CPMCU_STATIC_SCRATCH_FLOATS * 4 bytes until the
// process ends).
//
//   cpmcu_attention_mfma_static(...)  =  cpmcu_attention_mfma(...) without part_o / part_ml
//
// * Inputs and outputs are the caller's, as before: q, out [n, heads * head_dim] bf16, the paged key and
//   value pools, page table, positions, token slots, optional block lists.
// * It calls no hipMalloc, hipFree or allocating library routine.  Its first call on a device asks the
//   runtime for that device's address of the array (hipGetSymbolAddress), with that device current; later
//   calls only launch kernels on `stream`, which must belong to the current device.  That first call may
//   make the runtime load the library's code and takes a lock: a caller that captures a graph makes one call
//   on the device OUTSIDE any capture first (the runtime may refuse such calls under capture or end the
//   capture); the calls it then records only launch kernels.
// * n * heads * n_splits * (head_dim + 2) floats of shares must fit into the array; a larger call is refused
//   with a message that names the sizes, and nothing is launched.
// * All calls on one GPU share that GPU's array.  It keeps the last call's contents; nothing in it has to
//   start at zero (every share is written before it is read).  Calls that overlap on one GPU (two streams, two
//   threads) race on it: a caller must order them.
// * Returns nullptr, or a message valid until the calling thread's next call into the library.
#pragma once
#include <hip/hip_runtime.h>

// 4 Mi floats = 16 MiB: 64 tokens x 32 heads x 8 shares x (128 + 2), or 8 tokens x 32 heads x 64 shares
#define CPMCU_STATIC_SCRATCH_FLOATS (4 * 1024 * 1024)

extern "C" const char* cpmcu_attention_mfma_static(const void* q, void* out, int n, int nh, int nkv, int hd,
                                                   float scale, const void* kpool, const void* vtpool,
                                                   const int* page_table, int table_width, int page_size,
                                                   const int* positions, const int* tok_slot, const int* sel_blocks,
                                                   const int* sel_count, int max_sel, int block_size, int n_splits,
                                                   int waves_per_group, int last_blocks_first, hipStream_t stream);
