// Causal attention of a step's query tokens over the paged cache.
#pragma once
#include "common.h"

struct AttnArgs {
    int n_tokens, n_heads, n_kv_heads, head_dim;
    int page_size, table_width, num_pages;
    int q_stride, out_stride;  // elements between tokens
    int window;                // 0: all keys up to the query's position
    float scale;
};

#if defined(__HIPCC__)
// A step's entries bring their tokens as tiles of `per` tokens that never cross an entry; entries with one token
// bring none when the caller splits those by key range instead.  Which entry holds tile `tile`, and which of that
// entry's tiles it is: a wave finds out together, 64 entries at a time (a serving step has hundreds of entries,
// and a walk from entry to entry by every block cost a prompt portion's kernel more than its own work: 102 ->
// 182 us beside 230 decoding requests).  All lanes of a wave call these with the same arguments and get the same
// answers; false when the tile lies beyond the last one.
__device__ __forceinline__ int tiles_of_entry(const int* __restrict__ q_starts, int n_entries, int i, int per, int skip_single) {
    if (i >= n_entries) return 0;
    int cnt = q_starts[i + 1] - q_starts[i];
    return (cnt == 1 && skip_single) ? 0 : (cnt + per - 1) / per;
}
__device__ __forceinline__ int count_tiles(const int* __restrict__ q_starts, int n_entries, int per, int skip_single) {
    int lane = threadIdx.x & 63, mine = 0;
    for (int i = lane; i < n_entries; i += 64) mine += tiles_of_entry(q_starts, n_entries, i, per, skip_single);
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) mine += __shfl_xor(mine, d);
    return mine;
}
__device__ __forceinline__ bool locate_tile(const int* __restrict__ q_starts, int n_entries, int per, int skip_single,
                                            int tile, int& entry, int& within) {
    int lane = threadIdx.x & 63, left = tile;
    for (int base = 0; base < n_entries; base += 64) {
        int nt = tiles_of_entry(q_starts, n_entries, base + lane, per, skip_single);
        int incl = nt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int v = __shfl_up(incl, d);
            if (lane >= d) incl += v;
        }
        int total = __shfl(incl, 63);
        if (left < total) {
            unsigned long long holds = __ballot(left >= incl - nt && left < incl);    // one lane: its entry has tiles, and this one
            int src = __ffsll((long long)holds) - 1;
            entry = base + src;
            within = left - __shfl(incl - nt, src);
            return true;
        }
        left -= total;
    }
    return false;
}
#endif

// The matrix-core kernels (attention_mfma.hip).  Return 1 when they took the
// call, 0 when its shape is not theirs, -1 on error.
int llmrs_attention_bf16_mfma(hipStream_t stream, const bf16* q, bf16* out, const bf16* k_cache, const bf16* v_cache,
                              const int* block_table, const int* token_entry, const int* positions,
                              const int* q_starts, const int* seq_lens, int n_entries, float* scratch,
                              size_t scratch_bytes, int max_seq_len, int n_single, long single_keys, const AttnArgs& a);

// Keys per wave when the matrix-core kernels split `singles` single-token entries of up to max_seq_len keys
// that see single_keys keys together (0: unknown; 1 gives the smallest chunk any number of keys can give for these
// entries and this bound, which is what the scratch is sized by).
extern "C" int llmrs_attention_split_chunk(long singles, int n_kv_heads, int head_dim, int max_seq_len, long single_keys);

// 32-bit tiles on the matrix cores for entries with several tokens (attention_f32_mfma.hip); skip_single: entries
// with one token are left to the caller.  Return 1 when it took them, 0 when the shape is not its own, -1 on error.
int llmrs_attention_f32_mfma(hipStream_t stream, const float* q, float* out, const float* k_cache, const float* v_cache,
                             const int* block_table, const int* positions, const int* q_starts, int n_entries,
                             int skip_single, const AttnArgs& a);
// The same for entries with one token, split into chunks of F32_SPLIT_CHUNK keys whose partial results go to `partial`
// in the layout of attention_generic.hip's split, for that file's merge.
#define F32_SPLIT_CHUNK 128
int llmrs_attention_f32_mfma_split(hipStream_t stream, const float* q, float* partial, const float* k_cache, const float* v_cache,
                                   const int* block_table, const int* q_starts, const int* seq_lens, int n_entries,
                                   int max_chunks, const AttnArgs& a);
