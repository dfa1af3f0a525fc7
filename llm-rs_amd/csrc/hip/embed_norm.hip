// Token embedding into the 32-bit residual stream, and RMSNorm out of it.
#include "common.h"

typedef float embed_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 embed_bf16x8 __attribute__((ext_vector_type(8)));

// Eight values of a 16-bit row as one 16-byte load, widened and scaled (rows of a multiple of 8 values, 16-byte aligned).
__device__ __forceinline__ void load8_scaled(const bf16* src, float scale, float (&v)[8]) {
    embed_bf16x8 raw = *(const embed_bf16x8*)src;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (float)raw[j] * scale;
}
__device__ __forceinline__ void store8(float* dst, const float (&v)[8]) {
    *(embed_f32x4*)dst = embed_f32x4{v[0], v[1], v[2], v[3]};
    *(embed_f32x4*)(dst + 4) = embed_f32x4{v[4], v[5], v[6], v[7]};
}
template <class T>
__device__ __forceinline__ bool rows_by_eights(const T* table, const float* out, int D) {
    return sizeof(T) == 2 && D % 8 == 0 && ((uintptr_t)table & 15) == 0 && ((uintptr_t)out & 15) == 0;
}

// out[t, :] = float(table[tokens[t], :]) * scale   (reference: embed_batch_*, shaders/ops.metal:878-915,
// which has no scale: 1 there and for every architecture that does not ask for one)
template <class T>
__global__ void embed_rows_kernel(float* __restrict__ out, const T* __restrict__ table,
                                  const int* __restrict__ tokens, int D, int V, float scale) {
    int t = blockIdx.x;
    int row = tokens[t];
    row = row < 0 ? 0 : (row >= V ? V - 1 : row);  // the host has checked ids; never read outside the table
    const T* src = table + (size_t)row * D;
    float* dst = out + (size_t)t * D;
    if constexpr (sizeof(T) == 2) {
        if (rows_by_eights(table, out, D)) {           // (the same in all threads)
            for (int d = threadIdx.x * 8; d < D; d += blockDim.x * 8) {
                float v[8];
                load8_scaled((const bf16*)src + d, scale, v);
                store8(dst + d, v);
            }
            return;
        }
    }
    for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = to_f32(src[d]) * scale;
}

// One block per row: ss = sum x^2 in 32-bit, inv = 1/sqrt(ss/D + eps),
// y = (x * inv) * w, one rounding to the output type.  The weight multiplies
// directly (no 1+w).  Reference: rms_norm_batch, shaders/ops.metal:970-1003.
// The sum's order depends on D and the block size only, never on the row or batch.
template <class T>
__global__ void rmsnorm_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                    const float* __restrict__ w, const int* __restrict__ rows, int D, float eps) {
    __shared__ float partial[16];
    int r = rows ? rows[blockIdx.x] : blockIdx.x;
    const float* src = x + (size_t)r * D;
    float ss = 0.0f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float v = src[d];
        ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0) partial[wave] = ss;
    __syncthreads();
    float total = 0.0f;
    for (int i = 0; i < nwaves; ++i) total += partial[i];
    float inv = 1.0f / sqrtf(total / (float)D + eps);
    T* dst = out + (size_t)blockIdx.x * D;
    for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = from_f32<T>(src[d] * inv * w[d]);
}

// The same with the row held in registers between the sum and the scaling: one trip to
// memory instead of two, which is most of the time of a call with a few rows.  D % 4 == 0,
// D <= 4 * V4 * blockDim.  The sum's order again depends on D and the block size only.
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <class T, int V4>
__global__ void rmsnorm_rows_reg_kernel(T* __restrict__ out, const float* __restrict__ x,
                                        const float* __restrict__ w, const int* __restrict__ rows, int D, float eps) {
    __shared__ float partial[16];
    int r = rows ? rows[blockIdx.x] : blockIdx.x;
    const f32x4* src = (const f32x4*)(x + (size_t)r * D);
    int n4 = D / 4;
    f32x4 v[V4], ww[V4];
    float ss = 0.0f;
    // the norm's weight is asked for together with the row: a second trip to memory after the
    // sum would cost a call with few rows as much again as the first
#pragma unroll
    for (int i = 0; i < V4; ++i) {
        int idx = i * blockDim.x + threadIdx.x;
        v[i] = idx < n4 ? src[idx] : f32x4{0.f, 0.f, 0.f, 0.f};
        ww[i] = idx < n4 ? ((const f32x4*)w)[idx] : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < V4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) ss = fmaf(v[i][j], v[i][j], ss);
    ss = wave_sum(ss);
    int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0) partial[wave] = ss;
    __syncthreads();
    float total = 0.0f;
    for (int i = 0; i < nwaves; ++i) total += partial[i];
    float inv = 1.0f / sqrtf(total / (float)D + eps);
    T* dst = out + (size_t)blockIdx.x * D;
#pragma unroll
    for (int i = 0; i < V4; ++i) {
        int idx = i * blockDim.x + threadIdx.x;
        if (idx < n4) {
            if constexpr (sizeof(T) == 2) {       // four 16-bit results as one 8-byte store
                typedef T T4 __attribute__((ext_vector_type(4)));
                T4 o4;
#pragma unroll
                for (int j = 0; j < 4; ++j) o4[j] = from_f32<T>(v[i][j] * inv * ww[i][j]);
                *(T4*)(dst + idx * 4) = o4;
            } else {
                f32x4 o4;
#pragma unroll
                for (int j = 0; j < 4; ++j) o4[j] = v[i][j] * inv * ww[i][j];
                *(f32x4*)(dst + idx * 4) = o4;
            }
        }
    }
}

extern "C" int llmrs_embed_rows(hipStream_t stream, int dtype, float* out, const void* table, const int* tokens,
                                int n_tokens, int D, int V, float scale) {
    LLMRS_REQUIRE(n_tokens >= 0 && D > 0 && V > 0, "embed_rows: bad sizes T=%d D=%d V=%d", n_tokens, D, V);
    if (n_tokens == 0) return 0;
    if (dtype == LLMRS_F32)
        embed_rows_kernel<float><<<n_tokens, 256, 0, stream>>>(out, (const float*)table, tokens, D, V, scale);
    else if (dtype == LLMRS_BF16)
        embed_rows_kernel<bf16><<<n_tokens, 256, 0, stream>>>(out, (const bf16*)table, tokens, D, V, scale);
    else
        return llmrs_fail("embed_rows: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("embed_rows");
    return 0;
}

// rows == nullptr: row i of x -> row i of out; else row rows[i] of x -> row i of out.
extern "C" int llmrs_rmsnorm(hipStream_t stream, int dtype, void* out, const float* x, const float* weight,
                             const int* rows, int n_rows, int D, float eps) {
    LLMRS_REQUIRE(n_rows >= 0 && D > 0, "rmsnorm: bad sizes rows=%d D=%d", n_rows, D);
    LLMRS_REQUIRE(eps > 0.0f, "rmsnorm: eps must be positive, got %g", eps);
    if (n_rows == 0) return 0;
    if (dtype != LLMRS_F32 && dtype != LLMRS_BF16) return llmrs_fail("rmsnorm: unknown dtype %d", dtype);
    int threads = D > 4096 ? 1024 : 256;     // a row of up to 4096 fits the registers of four waves: fewer waves to start and to wait for
    bool in_registers = D % 4 == 0 && D <= 4 * 4 * threads && ((uintptr_t)x & 15) == 0 && ((uintptr_t)weight & 15) == 0 &&
                        ((uintptr_t)out & 15) == 0;
    if (in_registers && dtype == LLMRS_F32)
        rmsnorm_rows_reg_kernel<float, 4><<<n_rows, threads, 0, stream>>>((float*)out, x, weight, rows, D, eps);
    else if (in_registers)
        rmsnorm_rows_reg_kernel<bf16, 4><<<n_rows, threads, 0, stream>>>((bf16*)out, x, weight, rows, D, eps);
    else if (dtype == LLMRS_F32)
        rmsnorm_rows_kernel<float><<<n_rows, threads, 0, stream>>>((float*)out, x, weight, rows, D, eps);
    else
        rmsnorm_rows_kernel<bf16><<<n_rows, threads, 0, stream>>>((bf16*)out, x, weight, rows, D, eps);
    LLMRS_LAUNCH_CHECK("rmsnorm");
    return 0;
}
