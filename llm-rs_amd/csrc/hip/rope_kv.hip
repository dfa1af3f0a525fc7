// Rotary position encoding of q and k, and the write of k and v into the paged
// cache, in one pass over the projection's output.
//
// Rotation as the reference does it (rope_batch, shaders/ops.metal:1011-1042):
// angle = float(pos) * freq_i, (a, b) <- (a cos - b sin, a sin + b cos), all in
// 32-bit, one rounding on the way out.  freq_i comes from a table the host makes
// once (so that scaling of the frequencies is the host's matter); the pair is
// (i, i + rot/2) ("split half") or (2i, 2i+1) ("interleaved")
// (src/tensor/mod.rs:133-139).  Features past rotary_dim pass unchanged.
// The cache write replaces scatter_kv (shaders/ops.metal:841-853).
#include "cache_layout.h"
#include "common.h"
#include "gemm.h"

struct RopeKvArgs {
    int n_tokens, n_heads, n_kv_heads, head_dim;
    int rotary_dim, interleaved;
    int page_size, write_kv, num_pages;
    int row_stride;  // elements between tokens in qkv
    int value_pages; // the values of a page that 16 tokens fill in order are written whole, a kv head by each token's block
    // The projection's output still as the parts of its sum over k ([n_parts][n_tokens][n_cols], 32-bit), when the
    // product before was split over blocks and left the adding up to this kernel (null: the rows are in qkv).
    const float* parts;
    int n_parts, n_cols;
};

template <class T>
__global__ void rope_kv_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                               const int* __restrict__ slot_map, const float* __restrict__ inv_freq,
                               T* __restrict__ k_cache, T* __restrict__ v_cache, RopeKvArgs a) {
    int half = a.head_dim / 2;
    int pairs_per_token = (a.n_heads + 2 * a.n_kv_heads) * half;
    int t = blockIdx.x;
    int idx = blockIdx.y * blockDim.x + threadIdx.x;
    if (idx >= pairs_per_token) return;
    int head = idx / half, i = idx % half;
    T* row = qkv + (size_t)t * a.row_stride + (size_t)head * a.head_dim;
    bool is_q = head < a.n_heads;
    bool is_k = !is_q && head < a.n_heads + a.n_kv_heads;
    if (!is_q && !a.write_kv) return;
    int da, db;  // the two features this thread owns
    bool rotate = !(!is_q && !is_k) && i < a.rotary_dim / 2;
    if (i < a.rotary_dim / 2) {
        if (a.interleaved) { da = 2 * i; db = 2 * i + 1; }
        else { da = i; db = i + a.rotary_dim / 2; }
    } else {
        da = a.rotary_dim + 2 * (i - a.rotary_dim / 2);
        db = da + 1;
    }
    float xa = to_f32(row[da]), xb = to_f32(row[db]);
    if (rotate) {
        float angle = (float)positions[t] * inv_freq[i];
        float s, c;
        sincosf(angle, &s, &c);
        float ya = xa * c - xb * s;
        float yb = xa * s + xb * c;
        xa = ya; xb = yb;
    }
    if (is_q) {
        row[da] = from_f32<T>(xa);
        row[db] = from_f32<T>(xb);
        return;
    }
    int slot = slot_map[t];
    if (slot < 0 || slot >= a.num_pages * a.page_size) return;  // never write outside the cache
    int page = slot / a.page_size, off = slot % a.page_size;
    if (is_k) {
        int kvh = head - a.n_heads;
        k_cache[k_cache_index(page, kvh, off, da, a.n_kv_heads, a.page_size, a.head_dim)] = from_f32<T>(xa);
        k_cache[k_cache_index(page, kvh, off, db, a.n_kv_heads, a.page_size, a.head_dim)] = from_f32<T>(xb);
    } else {
        int kvh = head - a.n_heads - a.n_kv_heads;
        v_cache[v_cache_index(page, kvh, off, da, a.n_kv_heads, a.page_size, a.head_dim)] = from_f32<T>(xa);
        v_cache[v_cache_index(page, kvh, off, db, a.n_kv_heads, a.page_size, a.head_dim)] = from_f32<T>(xb);
    }
}

typedef __bf16 rope_bf16x8 __attribute__((ext_vector_type(8)));

// Values lie transposed in a page ([head_dim][slot]), so a token's values are head_dim scattered
// 2-byte stores.  Where 16 consecutive tokens of the batch fill one 16-slot page in order (a prompt
// portion, page after page), that page's values are written whole instead, the 16 tokens' blocks sharing out
// the kv heads: through LDS, 16 bytes a lane, whole lines.  All 16 blocks ask this of the same 16 tokens and get
// the same answer.  The first 16 lanes of a block's first wave look; the answer is the same in all of them.
__device__ __forceinline__ bool first_lanes_see_whole_page(const int* __restrict__ slot_map, int t16, const RopeKvArgs& a) {
    int j = threadIdx.x & 15;
    bool mine = false;
    if (a.page_size == 16 && t16 + 15 < a.n_tokens) {
        int s0 = slot_map[t16], sj = slot_map[t16 + j];
        mine = s0 >= 0 && (s0 & 15) == 0 && s0 + 15 < a.num_pages * 16 && sj == s0 + j;
    }
    return (__ballot(mine) & 0xffffull) == 0xffffull;
}

// Eight values of token t's row from column col on: from qkv, or added up from the parts of a split product, in
// the parts' order and rounded to 16 bits as the kernel that adds parts up rounds them (the same bits either way).
__device__ __forceinline__ rope_bf16x8 row_values(const bf16* __restrict__ qkv, int t, int col, const RopeKvArgs& a) {
    if (a.parts == nullptr) return *(const rope_bf16x8*)(qkv + (size_t)t * a.row_stride + col);
    const float* p = a.parts + (size_t)t * a.n_cols + col;
    size_t part = (size_t)a.n_tokens * a.n_cols;
    float4 lo = *(const float4*)p, hi = *(const float4*)(p + 4);
    for (int s = 1; s < a.n_parts; ++s) {
        float4 l2 = *(const float4*)(p + s * part), h2 = *(const float4*)(p + s * part + 4);
        lo.x += l2.x; lo.y += l2.y; lo.z += l2.z; lo.w += l2.w;
        hi.x += h2.x; hi.y += h2.y; hi.z += h2.z; hi.w += h2.w;
    }
    rope_bf16x8 v;
    v[0] = (bf16)lo.x; v[1] = (bf16)lo.y; v[2] = (bf16)lo.z; v[3] = (bf16)lo.w;
    v[4] = (bf16)hi.x; v[5] = (bf16)hi.y; v[6] = (bf16)hi.z; v[7] = (bf16)hi.w;
    return v;
}

// The values of 16 tokens that fill a page, for the kv heads first, first + 16, ...: [16 tokens][head_dim] in,
// [head_dim][16 slots] out, by all threads of a block, through `tile` ([16][head_dim + 8] in LDS).
__device__ __forceinline__ void write_value_page(const bf16* __restrict__ qkv, const int* __restrict__ slot_map,
                                                 bf16* __restrict__ v_cache, bf16* tile, int t16, int first,
                                                 const RopeKvArgs& a) {
    int hd = a.head_dim, ld = hd + 8, chunks = hd / 8;       // rows 16 bytes apart in banks
    int page = slot_map[t16] / 16;
    for (int kvh = first; kvh < a.n_kv_heads; kvh += 16) {
        int col = (a.n_heads + a.n_kv_heads + kvh) * hd;
        for (int c = threadIdx.x; c < 16 * chunks; c += blockDim.x) {
            int j = c / chunks, d0 = (c % chunks) * 8;
            *(rope_bf16x8*)(tile + j * ld + d0) = row_values(qkv, t16 + j, col + d0, a);
        }
        __syncthreads();
        bf16* dst = v_cache + v_cache_index(page, kvh, 0, 0, a.n_kv_heads, 16, hd);     // this page and head: [hd][16], contiguous
        for (int c = threadIdx.x; c < hd * 2; c += blockDim.x) {
            int d = c >> 1, s0 = (c & 1) * 8;
            rope_bf16x8 v;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = tile[(s0 + j) * ld + d];
            *(rope_bf16x8*)(dst + d * 16 + s0) = v;
        }
        __syncthreads();
    }
}

// The same for 16-bit rows whose pairs are neighbours (2i, 2i+1), eight features to a thread:
// one block per token works out the token's cos / sin once (they are the same for all of
// its heads) and then moves 16 bytes per thread and access.  Needs head_dim, rotary_dim and
// the row stride to be multiples of 8 and 16-byte aligned rows.
__global__ __launch_bounds__(256) void rope_kv_rows_kernel(bf16* __restrict__ qkv, const int* __restrict__ positions,
                                                           const int* __restrict__ slot_map,
                                                           const float* __restrict__ inv_freq,
                                                           bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
                                                           RopeKvArgs a) {
    extern __shared__ __attribute__((aligned(16))) float2 cs[];   // [rotary_dim / 2]: cos, sin of the token's angles; then a page's values
    __shared__ int values_elsewhere;               // this token's values are written with its page, the page's blocks sharing out the kv heads
    int t = blockIdx.x;
    if (threadIdx.x < 64) {
        bool w = a.write_kv && a.value_pages && first_lanes_see_whole_page(slot_map, t & ~15, a);
        if (threadIdx.x == 0) values_elsewhere = w;
    }
    float pos = (float)positions[t];
    for (int i = threadIdx.x; i < a.rotary_dim / 2; i += blockDim.x) {
        float s, c;
        sincosf(pos * inv_freq[i], &s, &c);
        cs[i] = float2{c, s};
    }
    __syncthreads();
    int slot = slot_map[t];
    bool cache_ok = a.write_kv && slot >= 0 && slot < a.num_pages * a.page_size;   // never write outside the cache
    int page = cache_ok ? slot / a.page_size : 0, off = cache_ok ? slot % a.page_size : 0;
    int chunks_per_head = a.head_dim / 8;
    int q_chunks = a.n_heads * chunks_per_head, all_chunks = (a.n_heads + 2 * a.n_kv_heads) * chunks_per_head;
    bf16* row = qkv + (size_t)t * a.row_stride;
    for (int ch = threadIdx.x; ch < all_chunks; ch += blockDim.x) {
        int head = ch / chunks_per_head, d0 = (ch % chunks_per_head) * 8;
        bool is_q = ch < q_chunks, is_k = !is_q && head < a.n_heads + a.n_kv_heads;
        if (!is_q && !cache_ok) continue;
        if (!is_q && !is_k && values_elsewhere) continue;
        rope_bf16x8 v = row_values(qkv, t, head * a.head_dim + d0, a);
        if ((is_q || is_k) && d0 < a.rotary_dim) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float2 w = cs[d0 / 2 + j];
                float xa = (float)v[2 * j], xb = (float)v[2 * j + 1];
                v[2 * j] = (bf16)(xa * w.x - xb * w.y);
                v[2 * j + 1] = (bf16)(xa * w.y + xb * w.x);
            }
        }
        if (is_q) {
            *(rope_bf16x8*)(row + (size_t)head * a.head_dim + d0) = v;
        } else if (is_k) {
            int kvh = head - a.n_heads;
            *(rope_bf16x8*)(k_cache + k_cache_index(page, kvh, off, d0, a.n_kv_heads, a.page_size, a.head_dim)) = v;
        } else {
            int kvh = head - a.n_heads - a.n_kv_heads;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                v_cache[v_cache_index(page, kvh, off, d0 + j, a.n_kv_heads, a.page_size, a.head_dim)] = v[j];
        }
    }
    if (values_elsewhere)                          // (the same in all threads of the block) the page's 16 blocks share out the kv heads
        write_value_page(qkv, slot_map, v_cache, (bf16*)(cs + (a.rotary_dim / 2 + 1) / 2 * 2), t & ~15, t & 15, a);
}

// Whether the kernel above (16-bit rows, pairs that are neighbours) takes these rows.
static bool rows_kernel_takes(const void* qkv, int row_stride, const void* k_cache, int n_tokens, int head_dim, int rotary_dim) {
    return n_tokens >= 16 && head_dim % 8 == 0 && rotary_dim % 8 == 0 && row_stride % 8 == 0 &&
           ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)k_cache & 15) == 0 && rotary_dim / 2 * sizeof(float2) <= 32768;
}
static void launch_rope_rows(hipStream_t stream, bf16* qkv, const int* positions, const int* slot_map, const float* inv_freq,
                             bf16* k_cache, bf16* v_cache, RopeKvArgs a) {
    a.value_pages = a.write_kv && a.page_size == 16 && a.n_kv_heads > 0 && ((uintptr_t)v_cache & 15) == 0 &&
                    (size_t)16 * (a.head_dim + 8) * 2 <= 32768;
    size_t smem = (size_t)(a.rotary_dim / 2 + 1) / 2 * 2 * sizeof(float2) + (a.value_pages ? (size_t)16 * (a.head_dim + 8) * 2 : 0);
    rope_kv_rows_kernel<<<a.n_tokens, 256, smem, stream>>>(qkv, positions, slot_map, inv_freq, k_cache, v_cache, a);
}

// qkv: [n_tokens, row_stride], a row is q heads, then k heads, then v heads.
// q is rotated in place; k is rotated and written to k_cache; v is copied to
// v_cache.  Slots outside [0, num_pages * page_size) are skipped.
extern "C" int llmrs_rope_kv_write(hipStream_t stream, int dtype, void* qkv, int row_stride, const int* positions,
                                   const int* slot_map, const float* inv_freq, int rotary_dim, int interleaved,
                                   void* k_cache, void* v_cache, int n_tokens, int n_heads, int n_kv_heads,
                                   int head_dim, int page_size, int num_pages, int write_kv) {
    LLMRS_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && head_dim > 0, "rope_kv_write: bad sizes");
    LLMRS_REQUIRE(head_dim % 2 == 0, "rope_kv_write: head_dim %d is odd", head_dim);
    LLMRS_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
                  "rope_kv_write: rotary_dim %d does not fit head_dim %d", rotary_dim, head_dim);
    LLMRS_REQUIRE(row_stride >= (n_heads + 2 * n_kv_heads) * head_dim, "rope_kv_write: row stride %d too short", row_stride);
    LLMRS_REQUIRE(page_size > 0, "rope_kv_write: page_size %d", page_size);
    if (n_tokens == 0) return 0;
    RopeKvArgs a{n_tokens, n_heads, n_kv_heads, head_dim, rotary_dim, interleaved, page_size, write_kv, num_pages, row_stride, 0,
                 nullptr, 0, 0};
    int pairs = (n_heads + 2 * n_kv_heads) * (head_dim / 2);
    dim3 grid(n_tokens, ceil_div(pairs, 256));
    if (dtype == LLMRS_F32)
        rope_kv_kernel<float><<<grid, 256, 0, stream>>>((float*)qkv, positions, slot_map, inv_freq, (float*)k_cache, (float*)v_cache, a);
    else if (dtype == LLMRS_BF16 && interleaved && rows_kernel_takes(qkv, row_stride, k_cache, n_tokens, head_dim, rotary_dim))
        launch_rope_rows(stream, (bf16*)qkv, positions, slot_map, inv_freq, (bf16*)k_cache, (bf16*)v_cache, a);
    else if (dtype == LLMRS_BF16)
        rope_kv_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)qkv, positions, slot_map, inv_freq, (bf16*)k_cache, (bf16*)v_cache, a);
    else
        return llmrs_fail("rope_kv_write: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("rope_kv_write");
    return 0;
}

extern "C" int llmrs_gemm(hipStream_t stream, int dtype, const void* A, int lda, const void* W, void* out, int ldc,
                          int M, int N, int K, int epi, void* workspace, size_t workspace_bytes, int allow_mfma,
                          const float* scale_sumsq, int scale_parts, float scale_eps, float* next_sumsq, void* next_y,
                          int next_ldy, const float* next_weight, float next_eps);

// qkv = x W^T for W = [q heads; k heads; v heads], then what llmrs_rope_kv_write does,
// with pairs (2i, 2i+1): in one kernel when the product is one the rotation fuses into
// (bfloat16, up to 64 tokens), else as two.  In the fused case only q is written to
// `qkv`; k and v go to the cache alone.
extern "C" int llmrs_qkv_rope_cache(hipStream_t stream, int dtype, const void* x, int lda, const void* w, void* qkv,
                                    int row_stride, int M, int K, const int* positions, const int* slot_map,
                                    const float* inv_freq, int rotary_dim, void* k_cache, void* v_cache,
                                    int n_heads, int n_kv_heads, int head_dim, int page_size, int num_pages,
                                    int write_kv, void* workspace, size_t workspace_bytes, int allow_mfma,
                                    const float* scale_sumsq, int scale_parts, float scale_eps) {
    // scale_sumsq: a norm left to this product (RowScale in gemm.h); then only the fused kernel will do
    int N = (n_heads + 2 * n_kv_heads) * head_dim;
    LLMRS_REQUIRE(M >= 0 && K > 0 && n_heads > 0 && n_kv_heads >= 0 && head_dim > 0, "qkv_rope_cache: bad sizes");
    LLMRS_REQUIRE(row_stride >= N && lda >= K, "qkv_rope_cache: row stride too short");
    LLMRS_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
                  "qkv_rope_cache: rotary_dim %d does not fit head_dim %d", rotary_dim, head_dim);
    LLMRS_REQUIRE(page_size > 0 && num_pages > 0, "qkv_rope_cache: bad cache geometry");
    if (M == 0) return 0;
    if (dtype == LLMRS_BF16 && allow_mfma) {
        QkvEpilogue qe{positions, slot_map, inv_freq, (bf16*)k_cache, (bf16*)v_cache, n_heads, n_kv_heads, head_dim,
                       rotary_dim, page_size, num_pages, write_kv};
        RowScale rs{scale_sumsq, scale_parts, scale_eps};
        int took = llmrs_gemm_bf16_mfma(stream, (const bf16*)x, lda, (const bf16*)w, qkv, row_stride, M, N, K,
                                        LLMRS_EPI_QKV, nullptr, 0, &qe, scale_sumsq ? &rs : nullptr);
        if (took != 0) return took < 0 ? -1 : 0;
        // A product that is split over blocks along k (65 to 512 rows, and some shapes from 17 rows on) leaves its parts:
        // the rotation kernel adds them up as it reads its rows, and the kernel that would do that is saved.
        if (scale_sumsq == nullptr && rows_kernel_takes(qkv, row_stride, k_cache, M, head_dim, rotary_dim) &&
            ((uintptr_t)workspace & 15) == 0 && N % 8 == 0) {
            int parts = llmrs_gemm_bf16_split_parts(stream, (const bf16*)x, lda, (const bf16*)w, M, N, K, workspace, workspace_bytes);
            if (parts < 0) return -1;
            if (parts > 1) {
                RopeKvArgs a{M, n_heads, n_kv_heads, head_dim, rotary_dim, 1, page_size, write_kv, num_pages, row_stride, 0,
                             (const float*)workspace, parts, N};
                launch_rope_rows(stream, (bf16*)qkv, positions, slot_map, inv_freq, (bf16*)k_cache, (bf16*)v_cache, a);
                LLMRS_LAUNCH_CHECK("qkv_rope_cache");
                return 0;
            }
        }
    }
    LLMRS_REQUIRE(scale_sumsq == nullptr, "qkv_rope_cache: a deferred norm needs the fused bfloat16 kernel (M=%d K=%d)", M, K);
    int rc = llmrs_gemm(stream, dtype, x, lda, w, qkv, row_stride, M, N, K, LLMRS_EPI_STORE, workspace, workspace_bytes,
                        allow_mfma, nullptr, 0, 0.0f, nullptr, nullptr, 0, nullptr, 0.0f);
    if (rc != 0) return rc;
    return llmrs_rope_kv_write(stream, dtype, qkv, row_stride, positions, slot_map, inv_freq, rotary_dim, 1, k_cache,
                               v_cache, M, n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv);
}
