// Shared by every kernel file: element types, the error channel of the C
// interface, launch checks.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

typedef __bf16 bf16;

enum LlmrsDtype { LLMRS_F32 = 0, LLMRS_BF16 = 1 };

// Message of the last failed call on this thread; read through llmrs_hip_error().
char* llmrs_error_buffer();
int llmrs_fail(const char* fmt, ...);
// Compute units of the current device (asked once; 256 if the device cannot be asked).
int llmrs_compute_units();

#define LLMRS_REQUIRE(cond, ...) \
    do {                         \
        if (!(cond)) return llmrs_fail(__VA_ARGS__); \
    } while (0)

#define LLMRS_LAUNCH_CHECK(name)                                              \
    do {                                                                      \
        hipError_t e_ = hipGetLastError();                                    \
        if (e_ != hipSuccess) return llmrs_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
    } while (0)

template <class T>
__device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <class T>
__device__ __forceinline__ T from_f32(float x) { return (T)x; }

// Four consecutive elements as 32-bit values: one 16-byte (float) or 8-byte (bfloat16) load.
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
    float4 t = *(const float4*)p;
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16* p, float (&v)[4]) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    bf16x4_t t = *(const bf16x4_t*)p;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (float)t[j];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// x / (1 + exp(-x)), as the reference writes it (shaders/ops.metal:769)
__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

static inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }
