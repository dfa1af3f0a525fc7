// Where a key or a value lies in a layer's part of the paged cache.
//
// Keys:   [page][kv_head][slot in page][head_dim]   a (page, head) is page_size rows of head_dim
// Values: [page][kv_head][head_dim][slot in page]   transposed, so that for one
//         feature the page's slots are contiguous: the PV product contracts over
//         keys, and the matrix cores want the contracted index contiguous.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>

__host__ __device__ __forceinline__ size_t k_cache_index(int page, int kv_head, int slot, int d,
                                                         int n_kv_heads, int page_size, int head_dim) {
    return (((size_t)page * n_kv_heads + kv_head) * page_size + slot) * head_dim + d;
}
__host__ __device__ __forceinline__ size_t v_cache_index(int page, int kv_head, int slot, int d,
                                                         int n_kv_heads, int page_size, int head_dim) {
    return (((size_t)page * n_kv_heads + kv_head) * head_dim + d) * page_size + slot;
}
