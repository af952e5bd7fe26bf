// Entry points of an attention library (attention_mfma.hip, built once per head size).  All return 0, or a
// negative code with the text in palm_last_error(); all validate on the host before they launch.
#pragma once

#include "common.h"

PALM_API int palm_attention_head_dim();
PALM_API int palm_attention_page_tokens();     // the cache's page size the library was built for

// One query a sequence over the paged cache.  With more than one slice of the key range the partial results
// (maximum, sum, unnormalised output of every slice) cross from the first kernel to the merging one through
// `work`: n_seqs * nh * n_slices * (hd + 4) floats of device memory that the caller brings.
PALM_API int palm_attention_decode(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                   const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                   int n_seqs, int nh, int nkv, int hd, float scale, int window, int n_slices,
                                   float* work, void* out);

// The same from the joined q/k/v projection's rows of the step's tokens (bfloat16 rows, or float32 planes of partial
// sums to be added): per-head RMS norm of q and k, rotation, the new key and value into the cache, attention.
PALM_API int palm_attention_decode_fused_serves(int rotary_dim, int pairing);
PALM_API int palm_attention_decode_fused(hipStream_t stream, const void* qkv, int qkv_is_planes, int planes,
                                         const float* q_norm_w, const float* k_norm_w, float eps, const float* cos_t,
                                         const float* sin_t, int rotary_dim, int pairing, int write_cache, void* k_cache,
                                         void* v_cache, const int* block_table, int max_pages, const int* seq_slot,
                                         const int* seq_start, int n_seqs, int nh, int nkv, int hd, float scale,
                                         int window, int n_slices, float* work, void* out);

// The same computation for callers that cannot allocate: code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose decode attention is a single
// kernel without a workspace, engine/cuda_attention.cu).  It takes no workspace: the slices' partial results go
// through a buffer that the library itself holds, a file-scope array in device memory of
// palm_attention_decode_static_limit() floats (8 MiB), which every GPU the library runs on keeps until the
// process ends.  The call allocates nothing, frees nothing and calls no allocating routine; it refuses
// n_seqs * nh * n_slices * (hd + 4) beyond the limit with an error and launches nothing then.  All calls on one
// GPU share that GPU's buffer, which keeps the last call's contents: nothing in it has to start at zero (every
// slice that holds keys writes its whole record before the merge reads it, and the merge reads no other), but two calls that overlap in
// time on one GPU (different streams, or a graph replayed beside an eager call) race on it.  Calls on one stream,
// one after the other, are safe.  The result is the same bits as palm_attention_decode's with the same slices.
PALM_API int palm_attention_decode_static(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                          const int* block_table, int max_pages, const int* seq_slot,
                                          const int* seq_start, int n_seqs, int nh, int nkv, int hd, float scale,
                                          int window, int n_slices, void* out);
PALM_API long long palm_attention_decode_static_limit();

// q_prescaled: the queries come multiplied by scale * log2(e) already and `scale` is not applied again; only where
// palm_attention_prefill_takes_prescaled() says so (the head sizes whose kernel gains from it).
PALM_API int palm_attention_prefill(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                    const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                    const int* seq_new, const int* cu_new, int n_seqs, int max_new, int nh, int nkv,
                                    int hd, float scale, int window, int q_prescaled, void* out);
PALM_API int palm_attention_prefill_takes_prescaled();
