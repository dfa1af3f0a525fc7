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
int llmrs_gemm_bf16_mfma(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                         int M, int N, int K, int epi, void* workspace, size_t workspace_bytes,
                         const QkvEpilogue* qkv = nullptr);
