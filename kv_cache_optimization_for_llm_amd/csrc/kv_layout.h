// Where a key lies inside a page of the K cache.
//
// A page of one kv head holds page_size keys of head_dim elements as [head_dim / C][page_size][C]:
// element `dim` of the key in row `row` of the page is at ((dim / C) * page_size + row) * C + dim % C,
// with C = 8 elements (16 bytes of bf16: what a lane of a matrix-core operand loads), or 4 where
// the head size is no multiple of 8.  The 16 keys x 32 dims a wavefront loads per product of S = K Q^T
// are then 1 KiB of neighbouring bytes - eight full cache lines - where keys laid out row by row
// give sixteen half-used ones.  (The reference keeps keys row by row inside a block,
// paged_attention/src/config.h:184-187, kernels.cu:175-176: its kernels walk a key with one thread.)
// V pages are stored transposed, [head_dim][page_size]: see rope_cache.hip.
#pragma once
#include <stddef.h>

__host__ __device__ inline int kva_k_chunk(int head_dim) { return (head_dim & 7) ? 4 : 8; }

// element offset inside the page of one kv head
__host__ __device__ inline size_t kva_k_at(int row, int dim, int page_size, int chunk) {
    return ((size_t)(dim / chunk) * page_size + row) * chunk + (dim % chunk);
}
