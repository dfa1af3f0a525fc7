// The plain product: 64x64 tiles through LDS, 32-bit FMA, k in ascending order.
// With the 32-bit matrix-core tiles and the few-row kernel below it is the whole
// 32-bit path (nothing here rounds its inputs) and the bfloat16 fallback for shapes
// the bfloat16 MFMA kernels refuse.  Within each of the three kernels the order of
// the sum for an output depends on K only, so a row's result does not depend on the
// row's place in the batch or on its tile; which kernel runs depends on M (up to 8
// rows, up to 16, more), so across those ranges results differ by rounding.
// Reference: gemm_f32 accumulates in 32-bit the same way (shaders/ops.metal:1053-1079).
#include "gemm.h"

#define TILE 64
#define TILE_K 16

template <class T>
__global__ __launch_bounds__(256) void gemm_simple_kernel(const T* __restrict__ A, int lda,
                                                          const T* __restrict__ W, void* __restrict__ out, int ldc,
                                                          int M, int N, int K, int epi) {
    __shared__ float As[TILE_K][TILE + 4];
    __shared__ float Ws[TILE_K][TILE + 4];
    int tid = threadIdx.x;
    int m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE;
    int ty = tid / 16, tx = tid % 16;
    int lrow = tid / 4, lk = (tid % 4) * 4;  // this thread stages 4 k-values of one row of each tile
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += TILE_K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int k = k0 + lk + i;
            int am = m0 + lrow, wn = n0 + lrow;
            As[lk + i][lrow] = (am < M && k < K) ? to_f32(A[(size_t)am * lda + k]) : 0.0f;
            Ws[lk + i][lrow] = (wn < N && k < K) ? to_f32(W[(size_t)wn * K + k]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TILE_K; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int m = m0 + ty * 4 + i;
        if (m >= M) continue;
        if (epi == LLMRS_EPI_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                int n = n0 + tx * 4 + j;
                if (n + 1 < N) ((T*)out)[(size_t)m * ldc + n / 2] = from_f32<T>(silu_f32(acc[i][j]) * acc[i][j + 1]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int n = n0 + tx * 4 + j;
                if (n < N) epilogue_store<T>(epi, out, ldc, m, n, acc[i][j]);
            }
        }
    }
}

// 32-bit products on the matrix cores: v_mfma_f32_32x32x2_f32 multiplies and adds in 32-bit (no
// reduced-precision mode), k in ascending order, so an output's sum depends on K only here too.
// 128 x 128 tiles of four waves (64 x 64 each), k in steps of 16 through two LDS buffers; the next
// step's rows are on their way to registers while this step is multiplied.  Any M, N, K: rows and
// k beyond the edges are read as zeros.
typedef float f32x16_t __attribute__((ext_vector_type(16)));
#define F32_BK 16
#define F32_LD (F32_BK + 1)      // LDS row stride in floats: lanes of an operand read (32 rows, one k each) hit distinct banks
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const float* __restrict__ A, int lda,
                                                            const float* __restrict__ W, void* __restrict__ out, int ldc,
                                                            int M, int N, int K, int epi) {
    __shared__ float As[2][128 * F32_LD];
    __shared__ float Ws[2][128 * F32_LD];
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave >> 1, wn = wave & 1;
    int m0 = blockIdx.y * 128, n0 = blockIdx.x * 128;
    // staging: thread t brings 4 consecutive k of rows (t / 4) and (t / 4 + 64) of each tile
    int srow = tid >> 2, sk = (tid & 3) * 4;
    const bool vec = K % 4 == 0 && lda % 4 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0;
    float ra[2][4], rw[2][4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int am = m0 + srow + 64 * h, wn_ = n0 + srow + 64 * h, k = k0 + sk;
            const float* ap = A + (size_t)min(am, M - 1) * lda + k;
            const float* wp = W + (size_t)min(wn_, N - 1) * K + k;
            if (vec && k + 3 < K) {
                load4(ap, ra[h]);
                load4(wp, rw[h]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    ra[h][j] = k + j < K ? ap[j] : 0.0f;
                    rw[h][j] = k + j < K ? wp[j] : 0.0f;
                }
            }
            if (am >= M)
#pragma unroll
                for (int j = 0; j < 4; ++j) ra[h][j] = 0.0f;
            if (wn_ >= N)
#pragma unroll
                for (int j = 0; j < 4; ++j) rw[h][j] = 0.0f;
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                As[buf][(srow + 64 * h) * F32_LD + sk + j] = ra[h][j];
                Ws[buf][(srow + 64 * h) * F32_LD + sk + j] = rw[h][j];
            }
    };
    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    int nk = (K + F32_BK - 1) / F32_BK;
    fetch(0);
    stage(0);
    __syncthreads();
    int frow = lane & 31, fk = lane >> 5;
    for (int kt = 0; kt < nk; ++kt) {
        int buf = kt & 1;
        if (kt + 1 < nk) fetch((kt + 1) * F32_BK);
        const float* as = As[buf] + (wm * 64 + frow) * F32_LD + fk;
        const float* ws = Ws[buf] + (wn * 64 + frow) * F32_LD + fk;
#pragma unroll
        for (int ks = 0; ks < F32_BK / 2; ++ks) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = as[i * 32 * F32_LD + ks * 2];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = ws[j * 32 * F32_LD + ks * 2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) stage(buf ^ 1);        // the other buffer's readers finished before the last barrier
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                float v = acc[i][j][r];
                if (epi == LLMRS_EPI_SWIGLU) {
                    float other = __shfl_xor(v, 1, 64);   // even lane: gate here, up next door
                    if (!(lane & 1) && m < M && n + 1 < N)
                        ((float*)out)[(size_t)m * ldc + n / 2] = silu_f32(v) * other;
                } else if (m < M && n < N) {
                    epilogue_store<float>(epi, out, ldc, m, n, v);
                }
            }
        }
}

// A few tokens (decoding): a wave for each pair of weight rows, every weight read once.
// Lanes stride over k, four elements at a time, and each keeps one 32-bit sum per token and
// row; the lanes' sums are added by a butterfly.  The order depends on K only.
#define GEMV_MAX_M 8
// VEC: K % 4 == 0 and every row starts on a multiple of four elements' size, so a lane's four
// elements come in one load and none of them lies past K.  RW weight rows per wave (even): the
// tokens' rows are read once for all of them.  The sums are the same whatever VEC and RW are.
template <class T, bool VEC, int RW>
__global__ __launch_bounds__(256) void gemm_rows_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W,
                                                        void* __restrict__ out, int ldc, int M, int N, int K, int epi) {
    int lane = threadIdx.x & 63;
    int n = RW * (blockIdx.x * 4 + (threadIdx.x >> 6));
    if (n >= N) return;
    const T* w[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) w[r] = W + (size_t)min(n + r, N - 1) * K;
    float acc[RW][GEMV_MAX_M] = {};
#pragma unroll 2
    for (int k = lane * 4; k < K; k += 256) {
        float a[RW][4];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            if constexpr (VEC) {
                load4(w[r] + k, a[r]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) a[r][j] = k + j < K ? to_f32(w[r][k + j]) : 0.0f;
            }
        }
#pragma unroll
        for (int m = 0; m < GEMV_MAX_M; ++m) {
            if (m >= M) break;
            const T* x = A + (size_t)m * lda + k;
            float xv[4];
            if constexpr (VEC) {
                load4(x, xv);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) xv[j] = k + j < K ? to_f32(x[j]) : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < RW; ++r) acc[r][m] = fmaf(a[r][j], xv[j], acc[r][m]);
        }
    }
#pragma unroll
    for (int m = 0; m < GEMV_MAX_M; ++m) {
        if (m >= M) break;
        float v[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) v[r] = wave_sum(acc[r][m]);
        if (lane != 0) continue;
#pragma unroll
        for (int r = 0; r < RW; r += 2) {
            if (epi == LLMRS_EPI_SWIGLU) {
                if (n + r + 1 < N) ((T*)out)[(size_t)m * ldc + (n + r) / 2] = from_f32<T>(silu_f32(v[r]) * v[r + 1]);
            } else {
                if (n + r < N) epilogue_store<T>(epi, out, ldc, m, n + r, v[r]);
                if (n + r + 1 < N) epilogue_store<T>(epi, out, ldc, m, n + r + 1, v[r + 1]);
            }
        }
    }
}

// Up to 16 tokens in 32-bit on the matrix cores: v_mfma_f32_16x16x4_f32 multiplies and adds in 32-bit (no
// reduced-precision mode).  The weight's rows are the A operand, read once, 16 bytes a lane (lane l: feature
// l % 16 of a tile, the four k-values 4 (l / 16) .. + 3 of a group of 16); the tokens' rows are the B operand, read
// the same way once for all of a block's NT feature tiles, so that the tokens cost a load for every NT loads of
// weights where the walk above asks for every token's row again for every two or four rows of the weight.  An MFMA
// contracts the four k-values that the four lane groups hold in the same place of their loads.  A block's NW waves
// take the 32-wide k-blocks in turn, U of them with all loads asked for before the first product, and add their sums
// through LDS in wave order: an output's sum depends on K (and on the weight's shape, which chooses NW) only.
// C: lane l holds token l % 16 and features 4 (l / 16) + r.  Needs K % 32 == 0 and 16-byte aligned rows.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
template <int NT, int NW, int U>
__global__ __launch_bounds__(NW * 64) void gemm_f32_skinny_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W,
                                                                  void* __restrict__ out, int ldc, int M, int N, int K, int epi) {
    extern __shared__ __attribute__((aligned(16))) float f32_skinny_red[];       // [NW][NT][4][64]
    float* red = f32_skinny_red;
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int row = lane & 15, g = lane >> 4;
    int n0 = blockIdx.x * NT * 16;
    const float* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wp[nt] = W + (size_t)min(n0 + nt * 16 + row, N - 1) * K + 4 * g;
    const float* xp = A + (size_t)min(row, M - 1) * lda + 4 * g;
    f32x4_t acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int nkb = K / 32;
    auto products = [&](const f32x4_t (&w)[NT][2], const f32x4_t (&x)[2]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[nt][half][j], x[half][j], acc[nt], 0, 0, 0);
    };
    int kb = wave;
    for (; kb + (U - 1) * NW < nkb; kb += U * NW) {
        f32x4_t w[U][NT][2], x[U][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int k = (kb + u * NW) * 32;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) { w[u][nt][0] = *(const f32x4_t*)(wp[nt] + k); w[u][nt][1] = *(const f32x4_t*)(wp[nt] + k + 16); }
            x[u][0] = *(const f32x4_t*)(xp + k);
            x[u][1] = *(const f32x4_t*)(xp + k + 16);
        }
        __builtin_amdgcn_sched_barrier(0);   // keep the round's loads together, ahead of its products
#pragma unroll
        for (int u = 0; u < U; ++u) products(w[u], x[u]);
    }
    for (; kb < nkb; kb += NW) {
        f32x4_t w[NT][2], x[2];
        int k = kb * 32;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) { w[nt][0] = *(const f32x4_t*)(wp[nt] + k); w[nt][1] = *(const f32x4_t*)(wp[nt] + k + 16); }
        x[0] = *(const f32x4_t*)(xp + k);
        x[1] = *(const f32x4_t*)(xp + k + 16);
        products(w, x);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((wave * NT + nt) * 4 + r) * 64 + lane] = acc[nt][r];
    __syncthreads();
    // the block's feature tiles are shared out over its waves; each is summed over the waves in order
    for (int nt = wave; nt < NT; nt += NW) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < NW; ++w2) s += red[((w2 * NT + nt) * 4 + r) * 64 + lane];
            v[r] = s;
        }
        int m = row, n = n0 + nt * 16 + 4 * g;
        if (m >= M) continue;
        if (epi == LLMRS_EPI_SWIGLU) {
#pragma unroll
            for (int r = 0; r < 4; r += 2)
                if (n + r + 1 < N) ((float*)out)[(size_t)m * ldc + (n + r) / 2] = silu_f32(v[r]) * v[r + 1];
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) epilogue_store<float>(epi, out, ldc, m, n + r, v[r]);
        }
    }
}

template <int NT, int NW, int U>
static void launch_f32_skinny(hipStream_t stream, const float* A, int lda, const float* W, void* out, int ldc, int M, int N, int K, int epi) {
    size_t bytes = (size_t)NW * NT * 4 * 64 * sizeof(float);
    static_assert((size_t)NW * NT * 4 * 64 * sizeof(float) <= 64 * 1024, "the waves' sums must fit in the LDS a block may ask for");
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)gemm_f32_skinny_kernel<NT, NW, U>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        configured = true;
    }
    gemm_f32_skinny_kernel<NT, NW, U><<<ceil_div(N, NT * 16), NW * 64, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
}

// A: [M, K] with row stride lda; W: [N, K] dense; out: row stride ldc (elements of
// its own type; for SWIGLU the output has N/2 columns).  workspace: optional device
// memory (16 * 64 * N * 4 bytes is always enough) for products that split K over blocks.
// scale_sumsq (with its parts and eps): a norm left to this product, see RowScale in gemm.h.  next_sumsq (with next_y,
// its row stride and the next norm's weight): what the += epilogue leaves for the norm that follows, see NextNorm.
// Both null in the ordinary case; otherwise the product must be one llmrs_gemm_defers_norm(M, N, K) accepts, in
// bfloat16 on the matrix cores, or the call fails.
extern "C" int llmrs_gemm(hipStream_t stream, int dtype, const void* A, int lda, const void* W, void* out, int ldc,
                          int M, int N, int K, int epi, void* workspace, size_t workspace_bytes, int allow_mfma,
                          const float* scale_sumsq, int scale_parts, float scale_eps, float* next_sumsq, void* next_y,
                          int next_ldy, const float* next_weight, float next_eps) {
    LLMRS_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    LLMRS_REQUIRE(lda >= K, "gemm: row stride %d of A is shorter than K=%d", lda, K);
    LLMRS_REQUIRE(epi >= 0 && epi <= 3, "gemm: unknown epilogue %d", epi);
    if (epi == LLMRS_EPI_SWIGLU) {
        LLMRS_REQUIRE(N % 2 == 0, "gemm: the gate/up epilogue needs an even N, got %d", N);
        LLMRS_REQUIRE(ldc >= N / 2, "gemm: row stride %d of out is shorter than N/2=%d", ldc, N / 2);
    } else {
        LLMRS_REQUIRE(ldc >= N, "gemm: row stride %d of out is shorter than N=%d", ldc, N);
    }
    if (M == 0) return 0;
    if (dtype == LLMRS_BF16 && allow_mfma) {
        RowScale rs{scale_sumsq, scale_parts, scale_eps};
        NextNorm nn{next_sumsq, (bf16*)next_y, next_ldy, next_weight, next_eps};
        int took = llmrs_gemm_bf16_mfma(stream, (const bf16*)A, lda, (const bf16*)W, out, ldc, M, N, K, epi, workspace,
                                        workspace_bytes, nullptr, scale_sumsq ? &rs : nullptr, next_y ? &nn : nullptr);
        if (took != 0) return took < 0 ? -1 : 0;
    }
    LLMRS_REQUIRE(scale_sumsq == nullptr && next_y == nullptr, "gemm: a deferred norm needs the bfloat16 matrix-core kernels (M=%d N=%d K=%d)", M, N, K);
    // (one or two tokens are better off with the walk below, which then asks for little beside the weights:
    // a decode step of the 8B shape at one request 7.1 against 7.8 ms)
    if (dtype == LLMRS_F32 && allow_mfma && M > 2 && M <= 16 && K % 32 == 0 && lda % 4 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0) {
        // (the waves per block follow the weight's shape alone, so a row's sums do not depend on the batch)
        const float* a = (const float*)A;
        const float* w = (const float*)W;
        // (blocks of 7 tiles with one wave a SIMD and one k-block in flight took 92 us for the 8B shape's gate/up
        // weight: a 32-bit MFMA is long, and the wave's loads and products took turns; two waves a SIMD, two k-blocks each)
        int cus = llmrs_compute_units();
        if (N >= 16384) {
            if (N % 112 == 0) launch_f32_skinny<7, 8, 2>(stream, a, lda, w, out, ldc, M, N, K, epi);
            else launch_f32_skinny<4, 4, 2>(stream, a, lda, w, out, ldc, M, N, K, epi);
        } else if (K >= 2048 && (ceil_div(N, 16) <= cus || ceil_div(N, 16) > 2 * cus)) launch_f32_skinny<1, 8, 4>(stream, a, lda, w, out, ldc, M, N, K, epi);
        // between one and two blocks a unit: blocks of four waves, two of which a unit holds side by side, make it one round
        else if (K >= 2048) launch_f32_skinny<1, 4, 8>(stream, a, lda, w, out, ldc, M, N, K, epi);
        else launch_f32_skinny<1, 4, 4>(stream, a, lda, w, out, ldc, M, N, K, epi);
        LLMRS_LAUNCH_CHECK("gemm");
        return 0;
    }
    if (M <= GEMV_MAX_M) {
        size_t elt = dtype == LLMRS_F32 ? sizeof(float) : sizeof(bf16);
        bool vec = K % 4 == 0 && lda % 4 == 0 && (uintptr_t)A % (4 * elt) == 0 && (uintptr_t)W % (4 * elt) == 0;
        // four weight rows per wave once several tokens share them, if that leaves six waves or more
        // for each compute unit (measured in 32-bit at 8 tokens: 28672 x 4096 130 -> 100 us; 4096 rows are
        // better off with two, 49 against 56 us)
        bool four = M > 2 && N >= 24 * llmrs_compute_units();
        int blocks = ceil_div(N, four ? 16 : 8);
#define ROWS(T, V) do { if (four) gemm_rows_kernel<T, V, 4><<<blocks, 256, 0, stream>>>((const T*)A, lda, (const T*)W, out, ldc, M, N, K, epi); \
                        else gemm_rows_kernel<T, V, 2><<<blocks, 256, 0, stream>>>((const T*)A, lda, (const T*)W, out, ldc, M, N, K, epi); } while (0)
        if (dtype == LLMRS_F32) { if (vec) ROWS(float, true); else ROWS(float, false); }
        else if (dtype == LLMRS_BF16) { if (vec) ROWS(bf16, true); else ROWS(bf16, false); }
        else return llmrs_fail("gemm: unknown dtype %d", dtype);
#undef ROWS
        LLMRS_LAUNCH_CHECK("gemm");
        return 0;
    }
    dim3 grid(ceil_div(N, TILE), ceil_div(M, TILE));
    LLMRS_REQUIRE(grid.y <= 65535, "gemm: M=%d is too large for one launch", M);
    if (dtype == LLMRS_F32 && allow_mfma && M > 16) {
        dim3 g128(ceil_div(N, 128), ceil_div(M, 128));
        LLMRS_REQUIRE(g128.y <= 65535, "gemm: M=%d is too large for one launch", M);
        gemm_f32_mfma_kernel<<<g128, 256, 0, stream>>>((const float*)A, lda, (const float*)W, out, ldc, M, N, K, epi);
    } else if (dtype == LLMRS_F32)
        gemm_simple_kernel<float><<<grid, 256, 0, stream>>>((const float*)A, lda, (const float*)W, out, ldc, M, N, K, epi);
    else if (dtype == LLMRS_BF16)
        gemm_simple_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)A, lda, (const bf16*)W, out, ldc, M, N, K, epi);
    else
        return llmrs_fail("gemm: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("gemm");
    return 0;
}
