// Attention with one wave for each (query token, head): the 32-bit path, and
// the bfloat16 path for head and page sizes the matrix-core kernel refuses.
//
// For the query at position p of its request, head h, kv head g = h / (heads per
// kv head): keys j = lo..p with lo = 0 or p + 1 - window; s_j = (q . k_j) * scale;
// softmax over j, computed online with a running maximum, all in 32-bit;
// o = sum_j softmax_j v_j, divided by the sum at the end.  The mask is the loop's
// bound.  This is the reference's paged_attention (shaders/ops.metal:636-758;
// causal_len of :673-674 equals p + 1) with a tile of 64 keys, one per lane.
// Tiles start at lo, so for a given query the order of every sum is fixed: it
// does not depend on the batch or on how the prompt was cut.
#include "attention.h"
#include "cache_layout.h"

#define MAX_HEAD_DIM 512

template <class T>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ token_entry, const int* __restrict__ positions,
    AttnArgs a) {
    __shared__ float qs[MAX_HEAD_DIM];
    int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    int hd = a.head_dim, ps = a.page_size;
    int kvh = h / (a.n_heads / a.n_kv_heads);
    int pos = positions[t];
    const int* table = block_table + (size_t)token_entry[t] * a.table_width;
    const T* qrow = q + (size_t)t * a.q_stride + (size_t)h * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();

    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    float m = -INFINITY, l = 0.0f;
    float acc[MAX_HEAD_DIM / 64] = {};
    for (int t0 = lo; t0 <= pos; t0 += 64) {
        int j = t0 + lane;
        bool valid = j <= pos;
        int page = 0, off = 0;
        float s = -INFINITY;
        if (valid) {
            page = table[min(j / ps, a.table_width - 1)];
            page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);  // stay inside the cache
            off = j % ps;
            const T* kp = k_cache + k_cache_index(page, kvh, off, 0, a.n_kv_heads, ps, hd);
            float dot = 0.0f;
            for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32(kp[d]), dot);
            s = dot * a.scale;
        }
        float m_new = fmaxf(m, wave_max(s));
        float p = valid ? expf(s - m_new) : 0.0f;
        float rescale = expf(m - m_new);
        l = l * rescale + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) acc[i] *= rescale;
        int n_valid = min(64, pos - t0 + 1);
        for (int jj = 0; jj < n_valid; ++jj) {
            float pj = __shfl(p, jj, 64);
            int pagej = __shfl(page, jj, 64), offj = __shfl(off, jj, 64);
#pragma unroll
            for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
                int d = lane + 64 * i;
                if (d < hd)
                    acc[i] = fmaf(pj, to_f32(v_cache[v_cache_index(pagej, kvh, offj, d, a.n_kv_heads, ps, hd)]), acc[i]);
            }
        }
    }
    T* orow = out + (size_t)t * a.out_stride + (size_t)h * hd;
#pragma unroll
    for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
        int d = lane + 64 * i;
        if (d < hd) orow[d] = from_f32<T>(acc[i] / l);
    }
}

// q: [n_tokens, q_stride] (head h at h*head_dim); out: [n_tokens, out_stride];
// block_table: [n_entries, table_width]; token_entry, positions: [n_tokens];
// q_starts: [n_entries+1], seq_lens: [n_entries].
// scratch: device memory for the partial results of single-token entries, which
// are split over waves by key range (may be null: then they are not split);
// max_seq_len: an upper bound of seq_lens that the host knows (0: unknown, no split);
// n_single: how many entries bring one token, if the host knows (-1: it does not).
extern "C" int llmrs_attention(hipStream_t stream, int dtype, const void* q, int q_stride, void* out, int out_stride,
                               const void* k_cache, const void* v_cache, const int* block_table, int table_width,
                               const int* token_entry, const int* positions, const int* q_starts,
                               const int* seq_lens, int n_entries, int n_tokens, int n_heads, int n_kv_heads,
                               int head_dim, int page_size, int num_pages, int window, float scale,
                               void* scratch, size_t scratch_bytes, int max_seq_len, int n_single, int allow_mfma) {
    LLMRS_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0, "attention: bad sizes");
    LLMRS_REQUIRE(n_heads % n_kv_heads == 0, "attention: %d heads are no multiple of %d kv heads", n_heads, n_kv_heads);
    LLMRS_REQUIRE(head_dim <= MAX_HEAD_DIM, "attention: head_dim %d exceeds %d", head_dim, MAX_HEAD_DIM);
    LLMRS_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0, "attention: bad cache geometry");
    LLMRS_REQUIRE(q_stride >= n_heads * head_dim && out_stride >= n_heads * head_dim, "attention: row stride too short");
    LLMRS_REQUIRE(window >= 0, "attention: negative window");
    LLMRS_REQUIRE(n_heads <= 65535, "attention: too many heads for one launch");
    if (n_tokens == 0) return 0;
    AttnArgs a{n_tokens, n_heads, n_kv_heads, head_dim, page_size, table_width, num_pages, q_stride, out_stride, window, scale};
    if (dtype == LLMRS_BF16 && allow_mfma) {
        int took = llmrs_attention_bf16_mfma(stream, (const bf16*)q, (bf16*)out, (const bf16*)k_cache, (const bf16*)v_cache,
                                             block_table, token_entry, positions, q_starts, seq_lens, n_entries,
                                             (float*)scratch, scratch_bytes, max_seq_len, n_single, a);
        if (took != 0) return took < 0 ? -1 : 0;
    }
    dim3 grid(n_tokens, n_heads);
    if (dtype == LLMRS_F32)
        attention_generic_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, (float*)out, (const float*)k_cache,
                                                                 (const float*)v_cache, block_table, token_entry, positions, a);
    else if (dtype == LLMRS_BF16)
        attention_generic_kernel<bf16><<<grid, 64, 0, stream>>>((const bf16*)q, (bf16*)out, (const bf16*)k_cache,
                                                                (const bf16*)v_cache, block_table, token_entry, positions, a);
    else
        return llmrs_fail("attention: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("attention");
    return 0;
}
