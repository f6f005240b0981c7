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

// The first key a query at position `pos` sees: 0, or - with a window - the window's start
// pos - window + 1, or - where positions see each other only inside chunks of `chunk` positions counted
// from 0 - the start of the query's own chunk.  (Keys past `pos` are never seen.)
__host__ __device__ inline int kva_first_visible(int pos, int window, int chunk) {
    if (chunk > 0) return pos - pos % chunk;
    return (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
}

// The same for kernels that take both masks in one number: `window` > 0 is a window of so many
// positions, `window` < 0 stands for chunks of -window positions, 0 for every earlier key.
__host__ __device__ inline int kva_first_visible_signed(int pos, int window) {
    return window < 0 ? pos - pos % (-window) : ((window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0);
}
