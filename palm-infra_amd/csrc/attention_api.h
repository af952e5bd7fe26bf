// Entry points of an attention library (attention_mfma.hip, built once per head size).  All return 0, or a
// negative code with the text in palm_last_error(); all validate on the host before they launch.
#pragma once

#include "common.h"

PALM_API int palm_attention_head_dim();

// One query a sequence over the paged cache.  With more than one slice of the key range the partial results
// (maximum, sum, unnormalised output of every slice) cross from the first kernel to the merging one through
// `work`: n_seqs * nh * n_slices * (hd + 4) floats of device memory that the caller brings.
PALM_API int palm_attention_decode(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                   const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                   int n_seqs, int nh, int nkv, int hd, float scale, int window, int n_slices,
                                   float* work, void* out);

PALM_API int palm_attention_prefill(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                    const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                    const int* seq_new, const int* cu_new, int n_seqs, int max_new, int nh, int nkv,
                                    int hd, float scale, int window, void* out);
