// bfloat16 products on the matrix cores, 32-bit accumulation.
//
// Two kernels, chosen by M (the number of tokens in the step):
//   M <= 32  "skinny": decoding.  Every weight is read once, straight from
//            memory into MFMA operands; a block owns 16 output features and its
//            waves split K, so a layer's product has enough waves in flight to
//            keep HBM busy.  v_mfma_f32_16x16x32_bf16, weights as the A operand.
//   M  > 32  "tiled": prompts.  128x128 (or 64x128) tiles of the output, K in
//            steps of 64 through double-buffered LDS, v_mfma_f32_32x32x16_bf16.
// Both need K % 8 == 0 and 16-byte aligned rows (16-byte loads); otherwise the
// caller falls back to the plain kernel.
//
// The order in which an output's products are summed depends on K, N and the
// kernel, never on M, the row's place in the batch or the tile it falls in.
// Replaces the reference's matvec_bf16_simd / gemm_bf16 (shaders/ops.metal:52-159,
// :1090-1143); unlike gemm_bf16 (:1107) the accumulator is 32-bit.
#include "gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *(const bf16x8*)p; }
__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16)0.0f;
    return z;
}

// ---------------------------------------------------------------------------
// skinny: C^T[n, m] = sum_k W[n, k] X[m, k]
//   A operand = W rows: lane l holds row n0 + l%16, 8 consecutive k
//   B operand = X rows: lane l holds token l%16 (+16 per tile), the same 8 k
//   C: lane l holds token l%16 and features n0 + 4*(l/16) + r, r = 0..3
// A lane's 8 k-values of one MFMA may be any 8, as long as both operands take
// the same; each lane group takes 16 consecutive k (two MFMAs), so that a wave
// reads 128 contiguous bytes of each of its 16 weight rows at a time.
// ---------------------------------------------------------------------------
template <int MT, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ A, int lda,
                                                              const bf16* __restrict__ W, void* __restrict__ out,
                                                              int ldc, int M, int N, int K, int epi) {
    __shared__ float red[NW][MT][4][64];
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int row = lane & 15, g = lane >> 4;
    int n0 = blockIdx.x * 16;
    const bf16* wp = W + (size_t)min(n0 + row, N - 1) * K;
    const bf16* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = A + (size_t)min(mt * 16 + row, M - 1) * lda;
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    int full = K / 64;             // blocks of 64 k that need no bounds
    int kb = wave;
#pragma unroll 4
    for (; kb < full; kb += NW) {
        int k = kb * 64 + g * 16;
        bf16x8 w0 = load8(wp + k), w1 = load8(wp + k + 8);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            bf16x8 x0 = load8(xp[mt] + k), x1 = load8(xp[mt] + k + 8);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc[mt], 0, 0, 0);
        }
    }
    if (kb == full && (K & 63)) {  // the wave whose turn it is takes the partial block
        int k = kb * 64 + g * 16;
        bool v0 = k < K, v1 = k + 8 < K;
        bf16x8 w0 = v0 ? load8(wp + k) : zero8(), w1 = v1 ? load8(wp + k + 8) : zero8();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            bf16x8 x0 = load8(xp[mt] + (v0 ? k : 0)), x1 = load8(xp[mt] + (v1 ? k + 8 : 0));
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc[mt], 0, 0, 0);
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][mt][r][lane] = acc[mt][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += red[w][mt][r][lane];  // waves in order: a fixed sum
            v[r] = s;
        }
        int m = mt * 16 + row;
        int n = n0 + 4 * g;
        if (m >= M) continue;
        if (epi == LLMRS_EPI_SWIGLU) {
#pragma unroll
            for (int r = 0; r < 4; r += 2)
                if (n + r + 1 < N) ((bf16*)out)[(size_t)m * ldc + (n + r) / 2] = (bf16)(silu_f32(v[r]) * v[r + 1]);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) epilogue_store<bf16>(epi, out, ldc, m, n + r, v[r]);
        }
    }
}

// ---------------------------------------------------------------------------
// tiled: C[m, n] = sum_k X[m, k] W[n, k]
//   A operand = X rows (lane l: row l%32, k-chunk l/32), B operand = W rows
//   C: lane l holds feature l%32 and tokens 8*(r/4) + 4*(l/32) + r%4, r = 0..15,
//   so a store instruction writes 32 consecutive features of a token.
// ---------------------------------------------------------------------------
#define BK 64
#define LDT (BK + 8)   // padded LDS row: 144 bytes, so 16 lanes' 16-byte reads hit distinct banks

template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ A, int lda,
                                                         const bf16* __restrict__ W, void* __restrict__ out,
                                                         int ldc, int M, int N, int K, int epi) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    bf16* smem = (bf16*)smem_raw;
    constexpr int TM = BM / 2, TN = BN / 2, FM = TM / 32, FN = TN / 32;
    constexpr int A_IT = BM / 32, W_IT = BN / 32, BUF = (BM + BN) * LDT;
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave >> 1, wn = wave & 1;
    int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int srow = tid >> 3, schunk = (tid & 7) * 8;   // staging: 8 threads per 128-byte row
    bf16x8 ra[A_IT], rw[W_IT];

    auto load_tile = [&](int kt) {
        int k = kt * BK + schunk;
        bool in = k < K;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) {
            int gm = min(m0 + srow + 32 * i, M - 1);
            ra[i] = in ? load8(A + (size_t)gm * lda + k) : zero8();
        }
#pragma unroll
        for (int i = 0; i < W_IT; ++i) {
            int gn = min(n0 + srow + 32 * i, N - 1);
            rw[i] = in ? load8(W + (size_t)gn * K + k) : zero8();
        }
    };
    auto store_tile = [&](int buf) {
        bf16* as = smem + buf * BUF;
        bf16* ws = as + BM * LDT;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) *(bf16x8*)(as + (srow + 32 * i) * LDT + schunk) = ra[i];
#pragma unroll
        for (int i = 0; i < W_IT; ++i) *(bf16x8*)(ws + (srow + 32 * i) * LDT + schunk) = rw[i];
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    int nk = (K + BK - 1) / BK;
    load_tile(0);
    store_tile(0);
    __syncthreads();
    int frow = lane & 31, fk = (lane >> 5) * 8;
    for (int kt = 0; kt < nk; ++kt) {
        int cur = kt & 1;
        if (kt + 1 < nk) load_tile(kt + 1);
        const bf16* as = smem + cur * BUF + (wm * TM + frow) * LDT + fk;
        const bf16* ws = smem + cur * BUF + BM * LDT + (wn * TN + frow) * LDT + fk;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 a[FM], b[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) a[i] = *(const bf16x8*)(as + i * 32 * LDT + ks * 16);
#pragma unroll
            for (int j = 0; j < FN; ++j) b[j] = *(const bf16x8*)(ws + j * 32 * LDT + ks * 16);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) store_tile(cur ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            int n = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                float v = acc[i][j][r];
                if (epi == LLMRS_EPI_SWIGLU) {
                    float other = __shfl_xor(v, 1, 64);   // even lane: gate here, up next door
                    if (!(lane & 1) && m < M && n + 1 < N)
                        ((bf16*)out)[(size_t)m * ldc + n / 2] = (bf16)(silu_f32(v) * other);
                } else if (m < M && n < N) {
                    epilogue_store<bf16>(epi, out, ldc, m, n, v);
                }
            }
        }
}

template <int BM, int BN>
static int launch_tiled(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                        int M, int N, int K, int epi) {
    static bool configured = false;
    size_t bytes = 2 * (BM + BN) * LDT * sizeof(bf16);
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<BM, BN>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return llmrs_fail("gemm: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
        configured = true;
    }
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM));
    if (grid.y > 65535) return llmrs_fail("gemm: M=%d is too large for one launch", M);
    gemm_tiled_kernel<BM, BN><<<grid, 256, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
    return 0;
}

int llmrs_gemm_bf16_mfma(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                         int M, int N, int K, int epi) {
    if (K % 8 || lda % 8 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return 0;
    int rc = 0;
    if (M <= 32) {
        // Waves per block from the weight's shape alone, so that a row's sum has one
        // order whatever the batch: 8 waves when K is long enough to share out.
        bool eight = K >= 2048;
        dim3 grid(ceil_div(N, 16));
        if (M <= 16) {
            if (eight) gemm_skinny_kernel<1, 8><<<grid, 512, 0, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
            else gemm_skinny_kernel<1, 4><<<grid, 256, 0, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
        } else {
            if (eight) gemm_skinny_kernel<2, 8><<<grid, 512, 0, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
            else gemm_skinny_kernel<2, 4><<<grid, 256, 0, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
        }
    } else if (M <= 64) {
        rc = launch_tiled<64, 128>(stream, A, lda, W, out, ldc, M, N, K, epi);
    } else {
        rc = launch_tiled<128, 128>(stream, A, lda, W, out, ldc, M, N, K, epi);
    }
    if (rc != 0) return -1;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        llmrs_fail("gemm (mfma): launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 1;
}
