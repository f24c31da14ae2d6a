// An entry point that allocates nothing.
//
// It has no counterpart in the reference (m87-labs/kestrel calls closed kernels and lets PyTorch
// allocate their workspaces). It is for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid `hipMalloc`.
//
// `ka_attention_decode_bf16_no_alloc` is `ka_attention_decode_bf16` without the `partial` /
// `partial_floats` arguments: decode attention over the paged cache, one token per row, the keys of
// a row cut into `splits` parts whose partial results a second kernel merges. The partial results
// go through a `static __device__` array inside the library, KA_NO_ALLOC_SCRATCH_FLOATS floats
// (4 MiB) that every GPU the library runs on holds until the process ends, instead of a buffer
// from the caller. The caller still passes every input and output. The call makes no `hipMalloc`,
// no `hipFree` and calls no allocating routine; the array's address on a device is looked up at
// the first call on that device (so make that call outside a graph capture).
//
// Limit: `n * H * splits * (hd + 2)` must not exceed KA_NO_ALLOC_SCRATCH_FLOATS when `splits > 1`
// (e.g. 64 tokens x 32 heads x 7 parts at head size 64); beyond that the call fails with -1 and
// `ka_last_error()` says so. With `splits == 1` the array is not used.
//
// All calls on one GPU share that GPU's array, which keeps the last call's contents. Nothing in it
// has to start at zero (every record read is written earlier in the same call), but two calls that
// overlap on one GPU (different streams, different threads) race on it: keep them on one stream
// or otherwise in order.
#pragma once

#include "ka_common.h"

constexpr long KA_NO_ALLOC_SCRATCH_FLOATS = 1L << 20;

// Arguments as `ka_attention_decode_bf16`, minus the scratch buffer and its size.
KA_API int ka_attention_decode_bf16_no_alloc(const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                                             const int* block_table, int max_pages, const int* token_row,
                                             const int* kv_lo, const int* kv_hi, void* out, long out_row_stride,
                                             float scale, int n, int H, int Hkv, int hd, int page_size, int splits,
                                             int waves, const void* k_new, const void* v_new, long new_stride,
                                             const float* table, int rot, const int* slots, void* k_cache_w,
                                             void* v_cache_w, hipStream_t stream);
