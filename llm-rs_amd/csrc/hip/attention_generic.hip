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
// does not depend on the batch or on how the prompt was cut.  A decoding request's
// keys are shared out over waves in chunks aligned to absolute positions and the
// chunks added in ascending order, which is another fixed order.
#include "attention.h"
#include "cache_layout.h"

#include <type_traits>

#define MAX_HEAD_DIM 512

// Keys of a single-token entry that one wave of the split takes (aligned to absolute positions).
#define GENERIC_CHUNK 128

// One wave walks the keys [begin, end) of its request for the query in `qs`, a tile of 64 keys at a
// time (one key per lane), and folds them into the running maximum m, sum l and acc (lane's
// features d = lane + 64 i, not yet divided by l).  VEC: head_dim % 4 == 0, a key's row is read four
// elements at a load; the sums are the same either way.
template <class T, bool VEC>
__device__ __forceinline__ void walk_keys(const float* qs, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                          const int* __restrict__ table, const AttnArgs& a, int kvh, int begin, int end,
                                          float& m, float& l, float (&acc)[MAX_HEAD_DIM / 64]) {
    int lane = threadIdx.x, hd = a.head_dim, ps = a.page_size;
    for (int t0 = begin; t0 < end; t0 += 64) {
        int j = t0 + lane;
        bool valid = j < end;
        int page = 0, off = 0;
        float s = -INFINITY;
        if (valid) {
            page = table[min(j / ps, a.table_width - 1)];
            page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);  // stay inside the cache
            off = j % ps;
            const T* kp = k_cache + k_cache_index(page, kvh, off, 0, a.n_kv_heads, ps, hd);
            float dot = 0.0f;
            if constexpr (VEC) {
                for (int d = 0; d < hd; d += 4) {
                    float kv[4];
                    load4(kp + d, kv);
#pragma unroll
                    for (int i = 0; i < 4; ++i) dot = fmaf(qs[d + i], kv[i], dot);
                }
            } else {
                for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32(kp[d]), dot);
            }
            s = dot * a.scale;
        }
        float m_new = fmaxf(m, wave_max(s));
        float p = valid ? expf(s - m_new) : 0.0f;
        float rescale = expf(m - m_new);
        l = l * rescale + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) acc[i] *= rescale;
        int n_valid = min(64, end - t0);
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
}

// skip_single: tokens of entries that bring one token are left to the split kernels below.
template <class T, bool VEC>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ token_entry, const int* __restrict__ positions,
    const int* __restrict__ q_starts, int skip_single, AttnArgs a) {
    __shared__ float qs[MAX_HEAD_DIM];
    int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    int hd = a.head_dim;
    int kvh = h / (a.n_heads / a.n_kv_heads);
    int e = token_entry[t];
    if (skip_single && q_starts[e + 1] - q_starts[e] == 1) return;
    int pos = positions[t];
    const int* table = block_table + (size_t)e * a.table_width;
    const T* qrow = q + (size_t)t * a.q_stride + (size_t)h * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();

    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    float m = -INFINITY, l = 0.0f;
    float acc[MAX_HEAD_DIM / 64] = {};
    walk_keys<T, VEC>(qs, k_cache, v_cache, table, a, kvh, lo, pos + 1, m, l, acc);
    T* orow = out + (size_t)t * a.out_stride + (size_t)h * hd;
#pragma unroll
    for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
        int d = lane + 64 * i;
        if (d < hd) orow[d] = from_f32<T>(acc[i] / l);
    }
}

// Entries with one token (decoding): a wave for each (entry, head, chunk of GENERIC_CHUNK keys), so
// that a long context is read by many waves at once.  Chunks are aligned to absolute positions.
// partial: [(entry * n_heads + head) * max_chunks + chunk][head_dim + 2] = m, l, acc (not divided).
template <class T, bool VEC>
__global__ __launch_bounds__(64) void attention_generic_split_kernel(
    const T* __restrict__ q, float* __restrict__ partial, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ q_starts, const int* __restrict__ seq_lens,
    int max_chunks, AttnArgs a) {
    __shared__ float qs[MAX_HEAD_DIM];
    int e = blockIdx.x, h = blockIdx.y, ch = blockIdx.z, lane = threadIdx.x;
    int t = q_starts[e];
    if (q_starts[e + 1] - t != 1) return;
    int pos = seq_lens[e] - 1;                    // an entry with one token: its position is its length less one
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    int first = lo / GENERIC_CHUNK;
    if (ch > pos / GENERIC_CHUNK - first) return;
    int begin = max(lo, (first + ch) * GENERIC_CHUNK), end = min(pos + 1, (first + ch + 1) * GENERIC_CHUNK);
    int hd = a.head_dim;
    int kvh = h / (a.n_heads / a.n_kv_heads);
    const T* qrow = q + (size_t)t * a.q_stride + (size_t)h * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();
    float m = -INFINITY, l = 0.0f;
    float acc[MAX_HEAD_DIM / 64] = {};
    walk_keys<T, VEC>(qs, k_cache, v_cache, block_table + (size_t)e * a.table_width, a, kvh, begin, end, m, l, acc);
    float* pp = partial + ((size_t)(e * a.n_heads + h) * max_chunks + ch) * (hd + 2);
    if (lane == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
    for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
        int d = lane + 64 * i;
        if (d < hd) pp[2 + d] = acc[i];
    }
}

// A wave that serves all G heads of a kv head reads a key or a value once for them; each head's sums
// are formed exactly as walk_keys forms them.  For 2, 4 or 8 heads per kv head and head sizes up
// to GROUP_MAX_HEAD_DIM.  qs: the G heads' queries side by side, [G][head_dim].
#define GROUP_MAX_HEAD_DIM 256
template <class T, bool VEC, int G>
__device__ __forceinline__ void walk_keys_group(const float* qs, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                const int* __restrict__ table, const AttnArgs& a, int kvh, int begin, int end,
                                                float (&m)[G], float (&l)[G], float (&acc)[G][GROUP_MAX_HEAD_DIM / 64]) {
    constexpr int NACC = GROUP_MAX_HEAD_DIM / 64;
    int lane = threadIdx.x, hd = a.head_dim, ps = a.page_size;
    for (int t0 = begin; t0 < end; t0 += 64) {
        int j = t0 + lane;
        bool valid = j < end;
        int page = 0, off = 0;
        float s[G];
#pragma unroll
        for (int g = 0; g < G; ++g) s[g] = -INFINITY;
        if (valid) {
            page = table[min(j / ps, a.table_width - 1)];
            page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);  // stay inside the cache
            off = j % ps;
            const T* kp = k_cache + k_cache_index(page, kvh, off, 0, a.n_kv_heads, ps, hd);
            float dot[G];
#pragma unroll
            for (int g = 0; g < G; ++g) dot[g] = 0.0f;
            if constexpr (VEC) {
                for (int d = 0; d < hd; d += 4) {
                    float kv[4];
                    load4(kp + d, kv);
#pragma unroll
                    for (int g = 0; g < G; ++g)
#pragma unroll
                        for (int i = 0; i < 4; ++i) dot[g] = fmaf(qs[g * hd + d + i], kv[i], dot[g]);
                }
            } else {
                for (int d = 0; d < hd; ++d) {
                    float kv = to_f32(kp[d]);
#pragma unroll
                    for (int g = 0; g < G; ++g) dot[g] = fmaf(qs[g * hd + d], kv, dot[g]);
                }
            }
#pragma unroll
            for (int g = 0; g < G; ++g) s[g] = dot[g] * a.scale;
        }
        float p[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float m_new = fmaxf(m[g], wave_max(s[g]));
            p[g] = valid ? expf(s[g] - m_new) : 0.0f;
            float rescale = expf(m[g] - m_new);
            l[g] = l[g] * rescale + wave_sum(p[g]);
            m[g] = m_new;
#pragma unroll
            for (int i = 0; i < NACC; ++i) acc[g][i] *= rescale;
        }
        int n_valid = min(64, end - t0);
        for (int jj = 0; jj < n_valid; ++jj) {
            int pagej = __shfl(page, jj, 64), offj = __shfl(off, jj, 64);
            float pj[G];
#pragma unroll
            for (int g = 0; g < G; ++g) pj[g] = __shfl(p[g], jj, 64);
#pragma unroll
            for (int i = 0; i < NACC; ++i) {
                int d = lane + 64 * i;
                if (d < hd) {
                    float v = to_f32(v_cache[v_cache_index(pagej, kvh, offj, d, a.n_kv_heads, ps, hd)]);
#pragma unroll
                    for (int g = 0; g < G; ++g) acc[g][i] = fmaf(pj[g], v, acc[g][i]);
                }
            }
        }
    }
}

// attention_generic_kernel with a wave for each (token, kv head).
template <class T, bool VEC, int G>
__global__ __launch_bounds__(64) void attention_generic_group_tokens_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ token_entry, const int* __restrict__ positions,
    const int* __restrict__ q_starts, int skip_single, AttnArgs a) {
    __shared__ float qs[G * GROUP_MAX_HEAD_DIM];
    constexpr int NACC = GROUP_MAX_HEAD_DIM / 64;
    int t = blockIdx.x, kvh = blockIdx.y, lane = threadIdx.x, hd = a.head_dim;
    int e = token_entry[t];
    if (skip_single && q_starts[e + 1] - q_starts[e] == 1) return;
    int pos = positions[t];
    const T* qrow = q + (size_t)t * a.q_stride + (size_t)kvh * G * hd;      // the kv head's G heads lie side by side
    for (int d = lane; d < G * hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    float m[G], l[G], acc[G][NACC];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY; l[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[g][i] = 0.0f;
    }
    walk_keys_group<T, VEC, G>(qs, k_cache, v_cache, block_table + (size_t)e * a.table_width, a, kvh, lo, pos + 1, m, l, acc);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        T* orow = out + (size_t)t * a.out_stride + (size_t)(kvh * G + g) * hd;
#pragma unroll
        for (int i = 0; i < NACC; ++i) {
            int d = lane + 64 * i;
            if (d < hd) orow[d] = from_f32<T>(acc[g][i] / l[g]);
        }
    }
}

// attention_generic_split_kernel with a wave for each (entry, kv head, chunk).
template <class T, bool VEC, int G>
__global__ __launch_bounds__(64) void attention_generic_group_kernel(
    const T* __restrict__ q, float* __restrict__ partial, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ q_starts, const int* __restrict__ seq_lens,
    int max_chunks, AttnArgs a) {
    __shared__ float qs[G * GROUP_MAX_HEAD_DIM];
    constexpr int NACC = GROUP_MAX_HEAD_DIM / 64;
    int e = blockIdx.x, kvh = blockIdx.y, ch = blockIdx.z, lane = threadIdx.x;
    int t = q_starts[e];
    if (q_starts[e + 1] - t != 1) return;
    int pos = seq_lens[e] - 1;                    // an entry with one token: its position is its length less one
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    int first = lo / GENERIC_CHUNK;
    if (ch > pos / GENERIC_CHUNK - first) return;
    int begin = max(lo, (first + ch) * GENERIC_CHUNK), end = min(pos + 1, (first + ch + 1) * GENERIC_CHUNK);
    int hd = a.head_dim;
    const T* qrow = q + (size_t)t * a.q_stride + (size_t)kvh * G * hd;
    for (int d = lane; d < G * hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();
    float m[G], l[G], acc[G][NACC];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY; l[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[g][i] = 0.0f;
    }
    walk_keys_group<T, VEC, G>(qs, k_cache, v_cache, block_table + (size_t)e * a.table_width, a, kvh, begin, end, m, l, acc);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float* pp = partial + ((size_t)(e * a.n_heads + kvh * G + g) * max_chunks + ch) * (hd + 2);
        if (lane == 0) { pp[0] = m[g]; pp[1] = l[g]; }
#pragma unroll
        for (int i = 0; i < NACC; ++i) {
            int d = lane + 64 * i;
            if (d < hd) pp[2 + d] = acc[g][i];
        }
    }
}

// One wave for each (entry, head) adds the chunks up.  The chunks' maxima and sums are read 64 at a time, a lane
// each; the weighted values are added chunk by chunk in ascending order, four chunks' rows asked for at a time.
template <class T>
__global__ __launch_bounds__(64) void attention_generic_merge_kernel(
    const float* __restrict__ partial, T* __restrict__ out, const int* __restrict__ q_starts,
    const int* __restrict__ seq_lens, int max_chunks, AttnArgs a) {
    int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, hd = a.head_dim;
    int t = q_starts[e];
    if (q_starts[e + 1] - t != 1) return;
    int pos = seq_lens[e] - 1;
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    int n_chunks = pos / GENERIC_CHUNK - lo / GENERIC_CHUNK + 1;
    const float* pp = partial + (size_t)(e * a.n_heads + h) * max_chunks * (hd + 2);
    const size_t stride = hd + 2;
    float M = -INFINITY;
    for (int ch = lane; ch < n_chunks; ch += 64) M = fmaxf(M, pp[(size_t)ch * stride]);
    M = wave_max(M);
    float L = 0.0f;
    float o[MAX_HEAD_DIM / 64] = {};
    for (int base = 0; base < n_chunks; base += 64) {
        int mine = base + lane;
        float w_mine = mine < n_chunks ? expf(pp[(size_t)mine * stride] - M) : 0.0f;
        float l_mine = mine < n_chunks ? pp[(size_t)mine * stride + 1] * w_mine : 0.0f;
        L += wave_sum(l_mine);
        int n = min(64, n_chunks - base);
        int j = 0;
        for (; j + 4 <= n; j += 4) {
            float v[4][MAX_HEAD_DIM / 64];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
                    int d = lane + 64 * i;
                    v[u][i] = d < hd ? pp[(size_t)(base + j + u) * stride + 2 + d] : 0.0f;
                }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float w = __shfl(w_mine, j + u, 64);
#pragma unroll
                for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) o[i] = fmaf(v[u][i], w, o[i]);
            }
        }
        for (; j < n; ++j) {
            float w = __shfl(w_mine, j, 64);
#pragma unroll
            for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
                int d = lane + 64 * i;
                if (d < hd) o[i] = fmaf(pp[(size_t)(base + j) * stride + 2 + d], w, o[i]);
            }
        }
    }
    T* orow = out + (size_t)t * a.out_stride + (size_t)h * hd;
#pragma unroll
    for (int i = 0; i < MAX_HEAD_DIM / 64; ++i) {
        int d = lane + 64 * i;
        if (d < hd) orow[d] = from_f32<T>(o[i] / L);
    }
}

// Room (in floats) for the partial results of the single-token entries (`singles` of n_entries, each of up to
// max_seq_len keys) that a call splits by key range: what the caller brings as scratch, whichever kernels take the call.
extern "C" long llmrs_attention_scratch_floats(int n_entries, int singles, int n_heads, int n_kv_heads, int head_dim,
                                               int max_seq_len) {
    if (max_seq_len <= 0 || n_entries <= 0 || n_heads <= 0 || n_kv_heads <= 0) return 0;
    int chunk = min(GENERIC_CHUNK, llmrs_attention_split_chunk(singles > 0 ? singles : n_entries, n_kv_heads, head_dim, max_seq_len, 1));
    return (long)n_entries * n_heads * ceil_div(max_seq_len, chunk) * (head_dim + 2);
}

template <class T>
static int launch_generic(hipStream_t stream, const T* q, T* out, const T* k_cache, const T* v_cache,
                          const int* block_table, const int* token_entry, const int* positions, const int* q_starts,
                          const int* seq_lens, int n_entries, float* scratch, size_t scratch_bytes, int max_seq_len,
                          int n_single, const AttnArgs& a, int allow_mfma) {
    bool vec = a.head_dim % 4 == 0 && (uintptr_t)k_cache % (4 * sizeof(T)) == 0;
    // Single-token entries are split by key range when the caller gave room for the partial results.
    int max_chunks = max_seq_len > 0 ? ceil_div(max_seq_len, GENERIC_CHUNK) : 0;
    size_t need = (size_t)n_entries * a.n_heads * max_chunks * (a.head_dim + 2) * sizeof(float);
    bool split = max_chunks > 0 && scratch != nullptr && q_starts != nullptr && seq_lens != nullptr &&
                 scratch_bytes >= need && n_single != 0 && n_entries <= 65535 && max_chunks <= 65535;
    bool only_single = split && n_single == n_entries && a.n_tokens == n_entries;     // every entry brings one token: the caller says so
    const int G = a.n_heads / a.n_kv_heads;
    const bool groupable = a.head_dim <= GROUP_MAX_HEAD_DIM && (G == 2 || G == 4 || G == 8);
    bool tiles_took = false;
    if constexpr (std::is_same<T, float>::value) {
        // 32-bit: entries with several tokens go to the matrix cores where the shape allows
        if (!only_single && allow_mfma) {
            int took = llmrs_attention_f32_mfma(stream, q, out, k_cache, v_cache, block_table, positions, q_starts, n_entries,
                                                split ? 1 : 0, a);
            if (took < 0) return -1;
            tiles_took = took == 1;
        }
    }
    if (!only_single && !tiles_took) {
        // a wave for all heads of a kv head when that still leaves two waves or more for each compute unit
        if (groupable && (long)a.n_tokens * a.n_kv_heads >= 2L * llmrs_compute_units()) {
            dim3 grid(a.n_tokens, a.n_kv_heads);
#define TOKENS(V, GG) attention_generic_group_tokens_kernel<T, V, GG><<<grid, 64, 0, stream>>>(q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, split, a)
            if (G == 8) { if (vec) TOKENS(true, 8); else TOKENS(false, 8); }
            else if (G == 4) { if (vec) TOKENS(true, 4); else TOKENS(false, 4); }
            else { if (vec) TOKENS(true, 2); else TOKENS(false, 2); }
#undef TOKENS
        } else {
            dim3 grid(a.n_tokens, a.n_heads);
            if (vec)
                attention_generic_kernel<T, true><<<grid, 64, 0, stream>>>(q, out, k_cache, v_cache, block_table, token_entry,
                                                                        positions, q_starts, split, a);
            else
                attention_generic_kernel<T, false><<<grid, 64, 0, stream>>>(q, out, k_cache, v_cache, block_table, token_entry,
                                                                         positions, q_starts, split, a);
        }
    }
    if (split) {
        static_assert(F32_SPLIT_CHUNK == GENERIC_CHUNK, "the matrix-core split leaves its chunks where this file's merge looks for them");
        bool mfma_took = false;
        if constexpr (std::is_same<T, float>::value) {
            // 32-bit: the single tokens' chunks on the matrix cores where the shape allows (one wave reads a chunk's keys
            // and values once for all heads of a kv head)
            if (allow_mfma) {
                int took = llmrs_attention_f32_mfma_split(stream, q, scratch, k_cache, v_cache, block_table, q_starts, seq_lens,
                                                          n_entries, max_chunks, a);
                if (took < 0) return -1;
                mfma_took = took == 1;
            }
        }
        // a wave for all heads of a kv head when that still leaves two waves or more for each compute unit
        // (measured in 32-bit at the 8B shape, 2048 keys: 8 requests 174 -> 88 us; one request alone is faster with a wave per head)
        long group_waves = (long)(n_single > 0 ? n_single : n_entries) * a.n_kv_heads * max_chunks;
        if (mfma_took) {
        } else if (groupable && group_waves >= 2L * llmrs_compute_units()) {
            dim3 grid(n_entries, a.n_kv_heads, max_chunks);
#define GROUP(V, GG) attention_generic_group_kernel<T, V, GG><<<grid, 64, 0, stream>>>(q, scratch, k_cache, v_cache, block_table, q_starts, seq_lens, max_chunks, a)
            if (G == 8) { if (vec) GROUP(true, 8); else GROUP(false, 8); }
            else if (G == 4) { if (vec) GROUP(true, 4); else GROUP(false, 4); }
            else { if (vec) GROUP(true, 2); else GROUP(false, 2); }
#undef GROUP
        } else {
            dim3 grid(n_entries, a.n_heads, max_chunks);
            if (vec)
                attention_generic_split_kernel<T, true><<<grid, 64, 0, stream>>>(q, scratch, k_cache, v_cache, block_table,
                                                                              q_starts, seq_lens, max_chunks, a);
            else
                attention_generic_split_kernel<T, false><<<grid, 64, 0, stream>>>(q, scratch, k_cache, v_cache, block_table,
                                                                               q_starts, seq_lens, max_chunks, a);
        }
        attention_generic_merge_kernel<T><<<dim3(n_entries, a.n_heads), 64, 0, stream>>>(scratch, out, q_starts, seq_lens,
                                                                                        max_chunks, a);
    }
    return 0;
}

// q: [n_tokens, q_stride] (head h at h*head_dim); out: [n_tokens, out_stride];
// block_table: [n_entries, table_width]; token_entry, positions: [n_tokens];
// q_starts: [n_entries+1], seq_lens: [n_entries].
// scratch: device memory for the partial results of single-token entries, which
// are split over waves by key range (may be null: then they are not split);
// max_seq_len: an upper bound of seq_lens that the host knows (0: unknown, no split);
// n_single: how many entries bring one token, if the host knows (-1: it does not); n_single == n_entries is the
// caller's word that every entry brings exactly one token (then token t is entry t, and q_starts is not read);
// single_keys: how many keys those entries see together (windows counted), if the host knows (0: it does not):
// the matrix-core kernels choose the keys per wave by it.
extern "C" int llmrs_attention(hipStream_t stream, int dtype, const void* q, int q_stride, void* out, int out_stride,
                               const void* k_cache, const void* v_cache, const int* block_table, int table_width,
                               const int* token_entry, const int* positions, const int* q_starts,
                               const int* seq_lens, int n_entries, int n_tokens, int n_heads, int n_kv_heads,
                               int head_dim, int page_size, int num_pages, int window, float scale,
                               void* scratch, size_t scratch_bytes, int max_seq_len, int n_single, long single_keys,
                               int allow_mfma) {
    LLMRS_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0, "attention: bad sizes");
    LLMRS_REQUIRE(n_heads % n_kv_heads == 0, "attention: %d heads are no multiple of %d kv heads", n_heads, n_kv_heads);
    LLMRS_REQUIRE(head_dim <= MAX_HEAD_DIM, "attention: head_dim %d exceeds %d", head_dim, MAX_HEAD_DIM);
    LLMRS_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0, "attention: bad cache geometry");
    LLMRS_REQUIRE(q_stride >= n_heads * head_dim && out_stride >= n_heads * head_dim, "attention: row stride too short");
    LLMRS_REQUIRE(window >= 0, "attention: negative window");
    LLMRS_REQUIRE(n_heads <= 65535, "attention: too many heads for one launch");
    LLMRS_REQUIRE(n_single <= n_entries, "attention: %d single-token entries among %d entries", n_single, n_entries);
    LLMRS_REQUIRE(n_single != n_entries || n_tokens == n_entries,
                  "attention: every entry is said to bring one token, but %d entries bring %d tokens", n_entries, n_tokens);
    if (n_tokens == 0) return 0;
    AttnArgs a{n_tokens, n_heads, n_kv_heads, head_dim, page_size, table_width, num_pages, q_stride, out_stride, window, scale};
    if (dtype == LLMRS_BF16 && allow_mfma) {
        int took = llmrs_attention_bf16_mfma(stream, (const bf16*)q, (bf16*)out, (const bf16*)k_cache, (const bf16*)v_cache,
                                             block_table, token_entry, positions, q_starts, seq_lens, n_entries,
                                             (float*)scratch, scratch_bytes, max_seq_len, n_single, single_keys, a);
        if (took != 0) return took < 0 ? -1 : 0;
    }
    int rc = 0;
    if (dtype == LLMRS_F32)
        rc = launch_generic<float>(stream, (const float*)q, (float*)out, (const float*)k_cache, (const float*)v_cache, block_table,
                                   token_entry, positions, q_starts, seq_lens, n_entries, (float*)scratch, scratch_bytes,
                                   max_seq_len, n_single, a, allow_mfma);
    else if (dtype == LLMRS_BF16)
        rc = launch_generic<bf16>(stream, (const bf16*)q, (bf16*)out, (const bf16*)k_cache, (const bf16*)v_cache, block_table,
                                  token_entry, positions, q_starts, seq_lens, n_entries, (float*)scratch, scratch_bytes,
                                  max_seq_len, n_single, a, allow_mfma);
    else
        return llmrs_fail("attention: unknown dtype %d", dtype);
    if (rc != 0) return -1;
    LLMRS_LAUNCH_CHECK("attention");
    return 0;
}
