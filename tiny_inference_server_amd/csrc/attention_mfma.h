// Entry points of the matrix-core attention library (attention_mfma.hip, built once per head size).
#pragma once
#include <hip/hip_runtime.h>

// floats of the workspace that tis_attention_mfma_static owns: 8 MiB on every GPU the library is used on
#define TIS_ATTENTION_STATIC_FLOATS (2 << 20)

extern "C" {

int tis_attention_mfma_head_dim();
int tis_attention_mfma_tile_columns();

// Attention of `rows` query rows over a paged cache plane. Partial results of split key ranges go to part_o / part_ml /
// row_splits, which the caller brings (see the comment above the definition for sizes and meanings).
int tis_attention_mfma(const void* q, long q_ld, const void* plane, const int* block_tables, int bt_ld,
                       const int* row_seq, const int* positions, const int* items, int n_items, int nb,
                       const int* tiles, int n_tiles, void* out, long out_ld, float* part_o, float* part_ml, int rows,
                       int n_heads, int n_kv_heads, int head_dim, int page_size, int window, float scale, int n_splits,
                       int min_steps, int tile_splits, int tile_max_steps, int* row_splits, hipStream_t stream);

// A second stream (default priority, as `stream` must have) on which a call that holds both tiles and items runs its
// tile kernel, beside the items' kernel on `stream`; the two meet again before the merge, and everything after the
// call on `stream` waits for both. Per device; null (the start) keeps everything on `stream`. The stream must outlive
// every later call on that device. Works under stream capture (the graph gets two branches).
int tis_attention_mfma_side_stream(hipStream_t side);

// The same attention for callers that cannot allocate device memory and have no workspace to bring: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference, whose
// attention kernels get their partial-result buffers from the tensor framework (paged_attention_kernels.py:229-231).
// Same arguments as tis_attention_mfma without the three workspace pointers; the same kernels run, so the results
// are the same. The partial results live in an array that the library itself holds on the device
// (TIS_ATTENTION_STATIC_FLOATS floats, for as long as the process lives). It allocates and frees nothing. A call
// whose partial results (rows x heads x splits x (head size + 2) + rows floats, splits being the larger of n_splits
// and tile_splits) do not fit is refused with a message; with one split nothing is needed and any size is taken.
// All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
// race on it and give wrong results; calls on one stream, one after the other, are fine. What a call leaves in the
// array means nothing to the next: every slot that is read has been written by the same call first.
int tis_attention_mfma_static(const void* q, long q_ld, const void* plane, const int* block_tables, int bt_ld,
                              const int* row_seq, const int* positions, const int* items, int n_items, int nb,
                              const int* tiles, int n_tiles, void* out, long out_ld, int rows, int n_heads,
                              int n_kv_heads, int head_dim, int page_size, int window, float scale, int n_splits,
                              int min_steps, int tile_splits, int tile_max_steps, hipStream_t stream);
long tis_attention_mfma_static_floats();
}
