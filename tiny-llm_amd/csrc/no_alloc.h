// An entry point that allocates nothing.
//
// It has no counterpart in the reference (zscey/tiny-llm), whose runtime plans one arena for all
// intermediates (tiny_llm/runtime/cuda/cuda_runtime.cpp:85-123).  It is for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.  `tl_flash_attention` splits a long context over workgroups and needs
// device memory beyond its inputs and outputs for the partial results
// ([n_splits, n_tokens, heads, head_dim + 2] float32), which its caller has to bring.
// `tl_flash_attention_static` is the same operation with the same kernels, but keeps the partial
// results in a device array that is part of the library: TL_STATIC_SCRATCH_FLOATS floats (4 MiB),
// held by every GPU the library runs on until the process ends.
//
//  * It calls no hipMalloc, hipFree or other allocating routine.  The first call on a device looks
//    the array's address up (hipGetSymbolAddress); make that call outside a graph capture.
//  * n_splits * n_tokens * heads * (head_dim + 2) must not exceed TL_STATIC_SCRATCH_FLOATS:
//    larger sizes return TL_ERR_SCRATCH and launch nothing.  With n_splits == 1 no scratch is used.
//  * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams,
//    two threads) race.  Calls on one stream are ordered and safe.  Nothing has to be cleared between
//    calls: every partial result that is read was written by the same call.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TL_STATIC_SCRATCH_FLOATS (1u << 20)
#define TL_ERR_SCRATCH 3   // the call needs more scratch than the library's static array holds

extern "C" {

// Arguments as tl_flash_attention, without part_o and part_ml.
int tl_flash_attention_static(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                              const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                              const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions,
                              void* out, int64_t out_stride, int n_tiles, int n_tokens, int nq, int nkv, int hd,
                              int block_size, float scale, int window, int n_splits, const float* rope_cos,
                              const float* rope_sin, int fuse_store, hipStream_t stream);

// The capacity of the static array, in floats.
int64_t tl_static_scratch_floats(void);

}
