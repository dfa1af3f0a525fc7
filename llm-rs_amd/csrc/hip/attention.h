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
