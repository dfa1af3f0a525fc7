// Next-token choice on the device: only token ids go back to the host.
#include "common.h"

// Greedy: the index of the largest logit; of equal ones the lowest index wins.
// (The reference's kernel, shaders/ops.metal:803-835, leaves ties to the scan's
// shape and its host path takes the last maximum, src/sampler/mod.rs:65-68; a
// rule is chosen here so that kernel and plain implementation agree.)
__device__ __forceinline__ void argmax_merge(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

__global__ __launch_bounds__(1024) void argmax_rows_kernel(const float* __restrict__ logits, int ld, int V,
                                                           int* __restrict__ out) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (size_t)blockIdx.x * ld;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        float v = row[i];
        if (v > best || idx == 0x7fffffff) { best = v; idx = i; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(best, off, 64);
        int oi = __shfl_xor(idx, off, 64);
        argmax_merge(best, idx, ov, oi);
    }
    int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { sv[wave] = best; si[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w) argmax_merge(best, idx, sv[w], si[w]);
        out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
    }
}

extern "C" int llmrs_argmax_rows(hipStream_t stream, const float* logits, int ld, int n_rows, int V, int* out) {
    LLMRS_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax_rows: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    if (n_rows == 0) return 0;
    argmax_rows_kernel<<<n_rows, 1024, 0, stream>>>(logits, ld, V, out);
    LLMRS_LAUNCH_CHECK("argmax_rows");
    return 0;
}
