// kva_attention_mfma_static: bf16 matrix-core attention over the paged cache that allocates
// nothing.
//
// This entry point has no counterpart in the reference.  It is for callers that cannot allocate
// device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  It is kva_attention_mfma (same arguments, same kernels, same results; one wavefront
// per key split) without the two buffers for the partial results of key splits: those live in a file-scope device array of
// KVA_ATTENTION_STATIC_SCRATCH_BYTES that every GPU the library runs on holds until the process
// ends.  The call makes no hipMalloc, hipFree or other allocating call; inputs and outputs are
// still the caller's.
//
// Limits and rules:
//   * kva_attention_mfma_static_scratch_bytes(total_rows, head_dim, splits) must not exceed
//     KVA_ATTENTION_STATIC_SCRATCH_BYTES (total_rows = tokens of the step x query heads); a
//     larger call is refused with an error that says so, nothing is launched;
//   * all calls on one GPU share that GPU's array, which keeps what the last call left in it;
//     nothing in it has to be cleared between calls (every partial that is read is written first
//     by the same call), but two calls that overlap in time on one GPU - on different streams, or
//     from different threads - race on it: serialise them;
//   * the array's device address is looked up once per device, at the first call made with that
//     device current.
#pragma once
#include <hip/hip_runtime.h>

#define KVA_ATTENTION_STATIC_SCRATCH_BYTES (16u << 20)

extern "C" long long kva_attention_mfma_static_scratch_bytes(int total_rows, int head_dim, int splits);

extern "C" int kva_attention_mfma_static(void *out, const void *q, int q_row_stride, const void *k_cache,
                                         const void *v_cache, const int *block_table, int max_blocks,
                                         const int *item_meta, const int *item_entry, const int *item_row0,
                                         int num_items, int row_tiles, const int *entry_seat,
                                         const int *entry_q_start, const int *entry_start_pos, int total_rows,
                                         int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                         float scale, int window, int splits, int keys_per_split, int pair,
                                         int all_rows, hipStream_t stream);
