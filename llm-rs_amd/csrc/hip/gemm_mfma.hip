// bfloat16 products on the matrix cores, 32-bit accumulation.
//
// Two kernels, chosen by M (the number of tokens in the step):
//   M <= 64  "skinny": decoding.  Every weight is read once, straight from
//            memory into MFMA operands; a block owns 16 to 64 output features and
//            its waves split K, so a layer's product has enough loads in flight to
//            keep HBM busy.  v_mfma_f32_16x16x32_bf16, weights as the A operand.
//   M  > 64  "tiled": prompts.  128x128 tiles of the output, K in steps of 64
//            through double-buffered LDS, v_mfma_f32_32x32x16_bf16.
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
//   A operand = W rows: lane l holds row n0 + l%16 (+16 per feature tile), 8 consecutive k
//   B operand = X rows: lane l holds token l%16 (+16 per token tile), the same 8 k
//   C: lane l holds token l%16 and features 4*(l/16) + r, r = 0..3
// A lane's 8 k-values of one MFMA may be any 8, as long as both operands take
// the same; of a block of 64 k, lane group g takes [8g, 8g+8) for one MFMA and
// [32+8g, 32+8g+8) for the next, so that each load instruction reads 64
// contiguous bytes of every row and the two together one 128-byte line.
// A block owns NT*16 features and MT*16 tokens; its NW waves take the 64-wide
// k-blocks in turn (wave w: w, w+NW, ...), U of them per round with all loads of
// a round issued before its first MFMA, and add their sums in wave order.
// ---------------------------------------------------------------------------
template <int MT, int NT, int NW, int U>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ A, int lda,
                                                              const bf16* __restrict__ W, void* __restrict__ out,
                                                              int ldc, int M, int N, int K, int epi) {
    extern __shared__ __attribute__((aligned(16))) unsigned char skinny_smem[];
    float* red = (float*)skinny_smem;          // [NW][MT][NT][4][64]
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int row = lane & 15, g = lane >> 4;
    int n0 = blockIdx.x * (NT * 16);
    const bf16* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wp[nt] = W + (size_t)min(n0 + nt * 16 + row, N - 1) * K;
    const bf16* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = A + (size_t)min(mt * 16 + row, M - 1) * lda;
    f32x4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

    int full = K / 64;             // blocks of 64 k that need no bounds
    int kb = wave;
    for (; kb + (U - 1) * NW < full; kb += U * NW) {
        bf16x8 w[U][NT][2], x[U][MT][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int k = (kb + u * NW) * 64 + g * 8;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) { w[u][nt][0] = load8(wp[nt] + k); w[u][nt][1] = load8(wp[nt] + k + 32); }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) { x[u][mt][0] = load8(xp[mt] + k); x[u][mt][1] = load8(xp[mt] + k + 32); }
        }
        __builtin_amdgcn_sched_barrier(0);   // keep the round's loads together, ahead of its MFMAs
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][nt][0], x[u][mt][0], acc[mt][nt], 0, 0, 0);
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][nt][1], x[u][mt][1], acc[mt][nt], 0, 0, 0);
                }
    }
    for (; kb <= full; kb += NW) {   // what is left of this wave's turns, and the partial block if it is its turn
        if (kb == full && !(K & 63)) break;
        int k = kb * 64 + g * 8;
        bool v0 = k < K, v1 = k + 32 < K;
        bf16x8 w0[NT], w1[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            w0[nt] = v0 ? load8(wp[nt] + k) : zero8();
            w1[nt] = v1 ? load8(wp[nt] + k + 32) : zero8();
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            bf16x8 x0 = load8(xp[mt] + (v0 ? k : 0)), x1 = load8(xp[mt] + (v1 ? k + 32 : 0));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[nt], x0, acc[mt][nt], 0, 0, 0);
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[nt], x1, acc[mt][nt], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[(((wave * MT + mt) * NT + nt) * 4 + r) * 64 + lane] = acc[mt][nt][r];
    __syncthreads();
    // the (mt, nt) tiles are shared out over the waves; each is summed over the waves in order
    for (int tile = wave; tile < MT * NT; tile += NW) {
        int mt = tile / NT, nt = tile % NT;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += red[(((w * MT + mt) * NT + nt) * 4 + r) * 64 + lane];
            v[r] = s;
        }
        int m = mt * 16 + row;
        int n = n0 + nt * 16 + 4 * g;
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

template <int MT, int NT, int NW, int U>
static void launch_skinny(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                          int M, int N, int K, int epi) {
    size_t bytes = (size_t)NW * MT * NT * 4 * 64 * sizeof(float);
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, NT, NW, U>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        configured = true;
    }
    gemm_skinny_kernel<MT, NT, NW, U><<<ceil_div(N, NT * 16), NW * 64, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
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
    if (M <= 64) {
        // Waves per block (NW) come from the weight's shape alone: k-blocks go to the
        // waves in turn and their sums are added in wave order, so for a given weight an
        // output's sum has one order whatever M, MT, NT and U are.
        // Features per block (NT*16) grow with N and M: a block reads its tokens' rows
        // again for every 16*NT features, which costs L2 bandwidth once M is large, but
        // a weight with few rows needs small blocks to have enough of them.
        // (Measured on MI355X at the 8B shapes; see profiles/.)
        bool wide = N >= 16384;
        bool eight = !wide && K >= 2048;
#define SKINNY(MT, NT, NW, U) launch_skinny<MT, NT, NW, U>(stream, A, lda, W, out, ldc, M, N, K, epi)
        if (M <= 16) {
            if (wide) { if (M <= 2) SKINNY(1, 1, 4, 8); else SKINNY(1, 4, 4, 2); }
            else if (eight) SKINNY(1, 1, 8, 4);
            else SKINNY(1, 1, 4, 4);
        } else if (M <= 32) {
            if (wide) SKINNY(2, 4, 4, 2);
            else if (N > 4096) { if (eight) SKINNY(2, 2, 8, 2); else SKINNY(2, 2, 4, 2); }
            else { if (eight) SKINNY(2, 1, 8, 4); else SKINNY(2, 1, 4, 4); }
        } else {
            if (wide) SKINNY(4, 4, 4, 2);
            else if (N > 4096) { if (eight) SKINNY(4, 2, 8, 1); else SKINNY(4, 2, 4, 2); }
            else { if (eight) SKINNY(4, 1, 8, 2); else SKINNY(4, 1, 4, 2); }
        }
#undef SKINNY
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
