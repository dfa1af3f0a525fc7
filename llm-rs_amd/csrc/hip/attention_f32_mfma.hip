// Causal attention of prompt portions in true 32-bit on the matrix cores:
// v_mfma_f32_32x32x2_f32 multiplies and adds in 32-bit (no reduced-precision mode),
// softmax in 32-bit as everywhere, probabilities never rounded.  It takes the place of the
// one-wave-per-token walk of attention_generic.hip for entries with several tokens when
// the engine computes in float32: a 2,048-token prompt is then bound by its products again.
//
// One wave owns 32 columns (the heads of one kv head for a few consecutive tokens of one
// request) and walks the keys it may see in tiles of 32, aligned to absolute positions:
//   S^T[key][col] = sum_d K[key][d] Q[col][d]        A operand = keys' rows, B = queries' rows
//   online softmax down each column (a lane holds 16 of a column's 32 keys, its partner
//   in the other half of the wave the other 16)
//   O^T[d][col] += sum_key V[key][d] P[key][col]      A = values, B = the probabilities where they stand
// An MFMA contracts two values, one from each half of the wave; which two is free as long as
// both operands agree.  For QK^T step (j, c) contracts d = 8j + c (lower half) and 8j + 4 + c
// (upper half), so a lane reads its row four consecutive values at a time; for PV step s
// contracts the two keys whose probabilities the two halves hold in register s of S^T, so the
// probabilities feed the second product without moving.  Values lie transposed in the cache,
// [feature][slot], so a lane reads four consecutive keys of its feature at a time.
// Needs head_dim % 32 == 0 (up to 256), page_size % 4 == 0, at most 32 heads per kv head,
// 16-byte aligned rows; otherwise the caller keeps to the walk.
// Entries with one token are shared out over waves by key range on the same products (attn_f32_split_kernel): a
// decode step in 32-bit reads its keys and values once for all heads of a kv head, 16 bytes a lane.
// Formulas: shaders/ops.metal:636-758 (scale after the dot, causal bound, softmax, weighted sum).
#include "attention.h"
#include "cache_layout.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float swap_halves(float x) {
    unsigned u = __float_as_uint(x);
    auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float((threadIdx.x & 32) ? sw[0] : sw[1]);
}

// One wave's walk over the keys [t_begin, t_end) (t_begin a multiple of 32) for its 32 columns: column c of this lane
// sees the keys lo..pos (pos < 0: a column that is not there).  Adds to the running maximum m (base 2, scale applied),
// the sum l and the sums O^T as they stand.
template <int HD>
__device__ __forceinline__ void f32_walk(const f32x4 (&qf)[HD / 8], const float* __restrict__ kc, const float* __restrict__ vc,
                                         const int* __restrict__ table, const AttnArgs& a, int kvh, int c, int h, int pos, int lo,
                                         int t_begin, int t_end, f32x16 (&O)[HD / 32], float& m, float& l) {
    const int ps = a.page_size;
    const float scale_log2e = a.scale * 1.44269504088896341f;     // exponentials in base 2: one multiply-add and one v_exp_f32
    auto page_of = [&](int key) {
        int pg = table[min(key / ps, a.table_width - 1)];
        return min(max(pg, 0), a.num_pages - 1);                   // stay inside the cache whatever the table holds
    };
    for (int t0 = t_begin; t0 < t_end; t0 += 32) {
        // the key this lane's A-operand row holds, and its row in the cache
        int key = t0 + c;
        const float* kp = kc + k_cache_index(page_of(key), kvh, key % ps, 4 * h, a.n_kv_heads, ps, HD);
        f32x4 kf[HD / 8];
#pragma unroll
        for (int j = 0; j < HD / 8; ++j) kf[j] = *(const f32x4*)(kp + 8 * j);
        // the values this lane's A-operand rows hold: feature dt * 32 + c, keys t0 + 8 g + 4 h .. + 3, g = 0..3.
        // Head sizes up to 128: all asked for now, so that their trip runs beside the first product; larger ones
        // (whose registers would not hold them all) one 32-feature tile at a time, right before its product.
        constexpr bool V_AHEAD = HD <= 128;
        const float* vp[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            int k0 = t0 + 8 * g + 4 * h;
            vp[g] = vc + v_cache_index(page_of(k0), kvh, k0 % ps, c, a.n_kv_heads, ps, HD);
        }
        f32x4 vf[V_AHEAD ? HD / 32 : 1][4];
        if constexpr (V_AHEAD) {
#pragma unroll
            for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) vf[dt][g] = *(const f32x4*)(vp[g] + (size_t)dt * 32 * ps);
        }
        f32x16 S;
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < HD / 8; ++j)
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) S = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[j][cc], qf[j][cc], S, 0, 0, 0);
        // register i of S holds the dot of this lane's column with key t0 + 8 (i / 4) + 4 h + i % 4
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int kk = t0 + 8 * (i >> 2) + 4 * h + (i & 3);
            S[i] = (kk > pos || kk < lo) ? -INFINITY : S[i] * scale_log2e;
            mx = fmaxf(mx, S[i]);
        }
        mx = fmaxf(mx, swap_halves(mx));
        float m_new = fmaxf(m, mx);
        float m_safe = m_new == -INFINITY ? 0.0f : m_new;          // a column that has seen no key yet
        float alpha = __builtin_amdgcn_exp2f(m - m_safe);          // (-inf - x: 0)
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            S[i] = __builtin_amdgcn_exp2f(S[i] - m_safe);
            sum += S[i];
        }
        sum += swap_halves(sum);
        l = l * alpha + sum;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) O[dt][i] *= alpha;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
            if constexpr (!V_AHEAD) {
#pragma unroll
                for (int g = 0; g < 4; ++g) vf[0][g] = *(const f32x4*)(vp[g] + (size_t)dt * 32 * ps);
            }
#pragma unroll
            for (int s = 0; s < 16; ++s)
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[V_AHEAD ? dt : 0][s >> 2][s & 3], S[s], O[dt], 0, 0, 0);
        }
    }
}

template <int HD>
__global__ __launch_bounds__(256) void attn_f32_tiles_kernel(const float* __restrict__ q, float* __restrict__ out,
                                                             const float* __restrict__ kc, const float* __restrict__ vc,
                                                             const int* __restrict__ block_table,
                                                             const int* __restrict__ positions,
                                                             const int* __restrict__ q_starts, int n_entries,
                                                             AttnArgs a, int G, int tpt, int skip_single) {
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int c = lane & 31, h = lane >> 5;
    int task = blockIdx.x * 4 + wave;
    int kvh = (task >> 2) % a.n_kv_heads;
    int tile = (task / (4 * a.n_kv_heads)) * 4 + (task & 3);
    int e = 0, rem = 0;
    if (!locate_tile(q_starts, n_entries, tpt, skip_single, tile, e, rem)) return;
    int tok0 = q_starts[e] + rem * tpt;
    int ntok = min(tpt, q_starts[e + 1] - tok0);
    int tq = c / G, hg = c - tq * G;
    bool cvalid = tq < ntok;
    int token = tok0 + min(tq, ntok - 1);
    int head = kvh * G + hg;
    int pos = cvalid ? positions[token] : -1;
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    int last = positions[tok0 + ntok - 1], first = positions[tok0];
    int t_end = last + 1;
    int t_begin = ((a.window > 0 && first + 1 > a.window) ? first + 1 - a.window : 0) & ~31;
    const int* table = block_table + (size_t)e * a.table_width;

    // this lane's part of its column's query: values 8j + 4h .. 8j + 4h + 3
    f32x4 qf[HD / 8];
    const float* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + 4 * h;
#pragma unroll
    for (int j = 0; j < HD / 8; ++j) qf[j] = *(const f32x4*)(qp + 8 * j);
    f32x16 O[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    f32_walk<HD>(qf, kc, vc, table, a, kvh, c, h, pos, lo, t_begin, t_end, O, m, l);
    if (!cvalid) return;
    float inv = 1.0f / l;
    float* op = out + (size_t)token * a.out_stride + (size_t)head * HD + 4 * h;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            f32x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = O[dt][4 * g + j] * inv;
            *(f32x4*)(op + dt * 32 + 8 * g) = v;
        }
}

// Entries with one token: a wave for each (entry, kv head, chunk of F32_SPLIT_CHUNK keys, aligned to absolute positions):
// its columns are the heads of the kv head (the other columns of the 32 multiply zeros: the keys and values are read
// once for all of them, 16 bytes a lane, which is what this step is bound by).  It leaves what the walk of
// attention_generic.hip leaves for such a chunk, where that file's merge finds it: the maximum (natural logarithm's
// scale), the sum and the weighted values of each head, [entry][head][chunk][2 + head_dim].
template <int HD>
__global__ __launch_bounds__(64) void attn_f32_split_kernel(const float* __restrict__ q, float* __restrict__ partial,
                                                            const float* __restrict__ kc, const float* __restrict__ vc,
                                                            const int* __restrict__ block_table,
                                                            const int* __restrict__ q_starts, const int* __restrict__ seq_lens,
                                                            int max_chunks, AttnArgs a, int G) {
    int lane = threadIdx.x, c = lane & 31, h = lane >> 5;
    int e = blockIdx.x, kvh = blockIdx.y, ch = blockIdx.z;
    int token = q_starts[e];
    if (q_starts[e + 1] - token != 1) return;
    int pos_t = seq_lens[e] - 1;                  // an entry with one token: its position is its length less one
    int lo = (a.window > 0 && pos_t + 1 > a.window) ? pos_t + 1 - a.window : 0;
    int first = lo / F32_SPLIT_CHUNK;
    if (ch > pos_t / F32_SPLIT_CHUNK - first) return;
    int begin = max(lo, (first + ch) * F32_SPLIT_CHUNK), end = min(pos_t + 1, (first + ch + 1) * F32_SPLIT_CHUNK);
    bool cvalid = c < G;
    int head = kvh * G + min(c, G - 1);
    int pos = cvalid ? pos_t : -1;
    const int* table = block_table + (size_t)e * a.table_width;
    f32x4 qf[HD / 8];
    const float* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + 4 * h;
#pragma unroll
    for (int j = 0; j < HD / 8; ++j) qf[j] = *(const f32x4*)(qp + 8 * j);
    f32x16 O[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    f32_walk<HD>(qf, kc, vc, table, a, kvh, c, h, pos, lo, begin & ~31, end, O, m, l);
    if (!cvalid) return;
    float* pp = partial + ((size_t)(e * a.n_heads + head) * max_chunks + ch) * (HD + 2);
    if (h == 0) { pp[0] = m * 0.69314718055994531f; pp[1] = l; }
    // this lane holds features dt * 32 + 8 g + 4 h + j of its column (rows of 2 + head_dim floats: 8-byte aligned)
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                float2 v = make_float2(O[dt][4 * g + j], O[dt][4 * g + j + 1]);
                *(float2*)(pp + 2 + dt * 32 + 8 * g + 4 * h + j) = v;
            }
}

// Takes the entries with several tokens (all entries when skip_single is 0).  Returns 1 when it took them,
// 0 when the shape is not its own (the caller then walks), -1 on error.
int llmrs_attention_f32_mfma(hipStream_t stream, const float* q, float* out, const float* k_cache, const float* v_cache,
                             const int* block_table, const int* positions, const int* q_starts, int n_entries,
                             int skip_single, const AttnArgs& a) {
    int G = a.n_heads / a.n_kv_heads;
    if (a.head_dim % 32 || a.head_dim > 256 || a.page_size % 4 || G > 32 || q_starts == nullptr) return 0;
    if (a.q_stride % 4 || a.out_stride % 4 || ((uintptr_t)q & 15) || ((uintptr_t)out & 15) || ((uintptr_t)k_cache & 15) ||
        ((uintptr_t)v_cache & 15))
        return 0;
    int tpt = 32 / G;
    long tiles = a.n_tokens / tpt + n_entries;
    long blocks = ((tiles + 3) / 4) * a.n_kv_heads;
    if (blocks > 0x7fffffffL) return 0;
    switch (a.head_dim) {
#define CASE(HD) case HD: attn_f32_tiles_kernel<HD><<<(int)blocks, 256, 0, stream>>>(q, out, k_cache, v_cache, block_table, positions, q_starts, n_entries, a, G, tpt, skip_single); break;
        CASE(32) CASE(64) CASE(96) CASE(128) CASE(160) CASE(192) CASE(224) CASE(256)
#undef CASE
        default: return 0;
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        llmrs_fail("attention (32-bit tiles): launch failed: %s", hipGetErrorString(err));
        return -1;
    }
    return 1;
}

// Takes the entries with one token, split by key range into `partial` (max_chunks chunks of F32_SPLIT_CHUNK keys an
// entry; the caller merges them).  Returns 1 when it took them, 0 when the shape is not its own, -1 on error.
int llmrs_attention_f32_mfma_split(hipStream_t stream, const float* q, float* partial, const float* k_cache, const float* v_cache,
                                   const int* block_table, const int* q_starts, const int* seq_lens, int n_entries,
                                   int max_chunks, const AttnArgs& a) {
    int G = a.n_heads / a.n_kv_heads;
    if (a.head_dim % 32 || a.head_dim > 256 || a.page_size % 4 || G > 32 || q_starts == nullptr || seq_lens == nullptr) return 0;
    if (a.q_stride % 4 || ((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || ((uintptr_t)partial & 7))
        return 0;
    if (n_entries > 65535 || a.n_kv_heads > 65535 || max_chunks > 65535 || max_chunks < 1) return 0;
    dim3 grid(n_entries, a.n_kv_heads, max_chunks);
    switch (a.head_dim) {
#define CASE(HD) case HD: attn_f32_split_kernel<HD><<<grid, 64, 0, stream>>>(q, partial, k_cache, v_cache, block_table, q_starts, seq_lens, max_chunks, a, G); break;
        CASE(32) CASE(64) CASE(96) CASE(128) CASE(160) CASE(192) CASE(224) CASE(256)
#undef CASE
        default: return 0;
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        llmrs_fail("attention (32-bit split): launch failed: %s", hipGetErrorString(err));
        return -1;
    }
    return 1;
}
