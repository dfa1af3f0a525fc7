// Small device utilities around the model: seeded normal fill (random-weights
// mode), dtype casts of whole tensors (weights on their way in), and the
// transform some architectures apply to their logits.
#include "../shared/normal_stream.h"
#include "common.h"

// out[i] = mean + std * normal_at(seed, first + i): the same bits as the host's
// llmrs_fill_normal_host for the same (seed, first + i).
template <class T>
__global__ void fill_normal_kernel(T* __restrict__ out, size_t n, uint64_t seed, uint64_t first, float mean, float std) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float v = llmrs::normal_value(seed, first + i, mean, std);
        if constexpr (sizeof(T) == 2) ((uint16_t*)out)[i] = llmrs::ns_bf16_bits(v);
        else out[i] = v;
    }
}

extern "C" int llmrs_fill_normal(hipStream_t stream, int dtype, void* out, size_t n, uint64_t seed, uint64_t first,
                                 float mean, float std) {
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "fill_normal: unknown dtype %d", dtype);
    if (n == 0) return 0;
    LLMRS_REQUIRE(out != nullptr, "fill_normal: null output");
    int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    if (dtype == LLMRS_F32) fill_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, n, seed, first, mean, std);
    else fill_normal_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)out, n, seed, first, mean, std);
    LLMRS_LAUNCH_CHECK("fill_normal");
    return 0;
}

// dst[i] = (D)src[i]; float16 and bfloat16 widen exactly, float32 -> bfloat16 rounds to nearest even.
enum { CAST_F32 = 0, CAST_BF16 = 1, CAST_F16 = 2 };

template <class S, class D>
__global__ void cast_kernel(D* __restrict__ dst, const S* __restrict__ src, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = (D)(float)src[i];
}

extern "C" int llmrs_cast(hipStream_t stream, void* dst, int dst_dtype, const void* src, int src_dtype, size_t n) {
    if (n == 0) return 0;
    LLMRS_REQUIRE(dst != nullptr && src != nullptr, "cast: null tensor");
    int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
#define CAST(S, D) cast_kernel<S, D><<<blocks, 256, 0, stream>>>((D*)dst, (const S*)src, n)
    if (src_dtype == CAST_F32 && dst_dtype == CAST_BF16) CAST(float, bf16);
    else if (src_dtype == CAST_F32 && dst_dtype == CAST_F32) CAST(float, float);
    else if (src_dtype == CAST_BF16 && dst_dtype == CAST_F32) CAST(bf16, float);
    else if (src_dtype == CAST_BF16 && dst_dtype == CAST_BF16) CAST(bf16, bf16);
    else if (src_dtype == CAST_F16 && dst_dtype == CAST_F32) CAST(_Float16, float);
    else if (src_dtype == CAST_F16 && dst_dtype == CAST_BF16) CAST(_Float16, bf16);
    else return llmrs_fail("cast: from dtype %d to dtype %d is not offered", src_dtype, dst_dtype);
#undef CAST
    LLMRS_LAUNCH_CHECK("cast");
    return 0;
}

// logits[r, v] <- logits[r, v] * scale, then, if cap > 0, cap * tanh(that / cap), in place and in 32-bit.
__global__ void scale_softcap_kernel(float* __restrict__ logits, int ld, int V, float scale, float cap) {
    float* row = logits + (size_t)blockIdx.y * ld;
    for (int v = blockIdx.x * blockDim.x + threadIdx.x; v < V; v += gridDim.x * blockDim.x) {
        float x = row[v] * scale;
        row[v] = cap > 0.0f ? cap * tanhf(x / cap) : x;
    }
}

extern "C" int llmrs_scale_softcap_rows(hipStream_t stream, float* logits, int ld, int n_rows, int V, float scale, float cap) {
    LLMRS_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "scale_softcap_rows: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    LLMRS_REQUIRE(cap >= 0.0f, "scale_softcap_rows: the cap must not be negative, got %g", cap);
    if (n_rows == 0) return 0;
    LLMRS_REQUIRE(n_rows <= 65535, "scale_softcap_rows: %d rows in one call (at most 65535)", n_rows);
    int bx = (V + 255) / 256 < 64 ? (V + 255) / 256 : 64;
    scale_softcap_kernel<<<dim3(bx, n_rows), 256, 0, stream>>>(logits, ld, V, scale, cap);
    LLMRS_LAUNCH_CHECK("scale_softcap_rows");
    return 0;
}
