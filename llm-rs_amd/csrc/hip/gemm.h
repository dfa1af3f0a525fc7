// C[m, n] = sum_k A[m, k] * W[n, k]: activations times a weight stored [out, in].
// What happens to the sum is the epilogue.
#pragma once
#include "common.h"

enum LlmrsEpilogue {
    LLMRS_EPI_STORE = 0,      // out[m, n] = acc, in the activation type
    LLMRS_EPI_STORE_F32 = 1,  // out[m, n] = acc, 32-bit (logits)
    LLMRS_EPI_ACCUM_F32 = 2,  // out[m, n] += acc, 32-bit (the residual stream)
    LLMRS_EPI_SWIGLU = 3,     // rows of W are (gate_0, up_0, gate_1, up_1, ...):
                              // out[m, n/2] = silu(acc[m, n]) * acc[m, n+1] for even n, activation type
    LLMRS_EPI_QKV = 4,        // rows of W are q heads, k heads, v heads: rotate q and k (adjacent pairs),
                              // q to out, k and v straight into the paged cache (QkvEpilogue)
};

// What the q/k/v epilogue needs beside the sums.
struct QkvEpilogue {
    const int* positions;     // [M]
    const int* slot_map;      // [M] page * page_size + slot
    const float* inv_freq;    // [rotary_dim / 2]
    bf16* k_cache;
    bf16* v_cache;
    int n_heads, n_kv_heads, head_dim, rotary_dim;
    int page_size, num_pages, write_kv;
};

// RMSNorm without a kernel of its own, for steps of up to 16 tokens.  The product that adds into the
// 32-bit stream (its last writer before a norm) also leaves, for the norm that follows,
//   y[m, n]     = bfloat16(h[m, n] * weight[n])        the new row times the norm's weight, rounded once
//   sumsq[m, p] = sum of h[m, n]^2 over the 16 (for some shapes 8) features n of group p
// (NextNorm); the product that follows takes y as its rows and multiplies each of its 32-bit sums by
//   inv[m] = 1 / sqrt(sum_p sumsq[m, p] / K + eps)       (RowScale; the groups are added in a fixed order)
// before its epilogue.  x W^T with x = h inv weight is the same number as inv (h weight) W^T; what
// differs from the norm kernel's output is where the one rounding to bfloat16 falls (on h weight
// instead of on h inv weight), not how many there are.
// With more rows, a product whose sums are split over blocks (k ranges) has a kernel that adds the parts up, and
// that kernel sees whole rows: with eps > 0 it finishes the following norm itself,
//   y[m, n] = bfloat16(h[m, n] * inv[m] * weight[n])
// which any product takes as plain rows (sumsq is not used then).
struct NextNorm {
    float* sumsq;          // [M, llmrs_gemm_next_parts(M, N, K)]: a part per 16 features, or per 8 (not used with eps > 0)
    bf16* y;               // [M, N], row stride ldy; null: nothing is left
    int ldy;
    const float* weight;   // [N]
    float eps;             // > 0: the norm is finished here (llmrs_gemm_norms_whole), else left to the next product
};
struct RowScale {
    const float* sumsq;    // [M, nparts]; null: no scale
    int nparts;
    float eps;
};

template <class T>
__device__ __forceinline__ void epilogue_store(int epi, void* out, int ldc, int m, int n, float v) {
    if (epi == LLMRS_EPI_STORE) ((T*)out)[(size_t)m * ldc + n] = from_f32<T>(v);
    else if (epi == LLMRS_EPI_STORE_F32) ((float*)out)[(size_t)m * ldc + n] = v;
    else if (epi == LLMRS_EPI_ACCUM_F32) ((float*)out)[(size_t)m * ldc + n] += v;
}

// The 16-byte-load kernels on MFMA (gemm_mfma.hip).  Return 1 when they took the
// product, 0 when its shape or alignment is not theirs, -1 on error.
// workspace: device memory for the partial sums of products that split K over blocks (may be null).
// qkv: needed when epi is LLMRS_EPI_QKV; such a call is taken only by the kernels that fuse it.
// scale, next: see RowScale and NextNorm; both only where llmrs_gemm_defers_norm(M, N, K) holds (next: with
// LLMRS_EPI_ACCUM_F32 only), or next with eps where llmrs_gemm_norms_whole(M, N, K) holds.
// The product left as the parts of its sum over k, [parts][M][N] 32-bit in `workspace` (gemm_mfma.hip): the number of
// parts, 0 when this product would not be split (nothing launched), -1 on error.
int llmrs_gemm_bf16_split_parts(hipStream_t stream, const bf16* A, int lda, const bf16* W, int M, int N, int K,
                                void* workspace, size_t workspace_bytes);
int llmrs_gemm_bf16_mfma(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                         int M, int N, int K, int epi, void* workspace, size_t workspace_bytes,
                         const QkvEpilogue* qkv = nullptr, const RowScale* scale = nullptr, const NextNorm* next = nullptr);
// Whether the bfloat16 product of this shape goes to the kernel that can scale its rows' sums and leave a NextNorm.
extern "C" int llmrs_gemm_defers_norm(int M, int N, int K);
// The parts per row of the sums of squares that such a product leaves (NextNorm): what the caller sizes sumsq by.
extern "C" int llmrs_gemm_next_parts(int M, int N, int K);
// Whether the bfloat16 product of this shape, adding into the stream and given the workspace that
// llmrs_gemm_workspace_floats asks for, is split over blocks so that it can finish the following norm (NextNorm with eps).
extern "C" int llmrs_gemm_norms_whole(int M, int N, int K);
