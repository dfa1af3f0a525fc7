// bfloat16 products on the matrix cores, 32-bit accumulation.
//
// Two kernels, chosen by M (the number of tokens in the step):
//   M <= 64  "skinny": decoding.  Every weight is read once, straight from
//            memory into MFMA operands; a block owns 16 to 64 output features and
//            its waves split K, so a layer's product has enough loads in flight to
//            keep HBM busy.  v_mfma_f32_16x16x32_bf16, weights as the A operand.
//   M  > 64  "tiled": prompts.  128x128 or 256x256 tiles of the output, K in steps
//            of 64 through double-buffered LDS, v_mfma_f32_32x32x16_bf16; the tiles are
//            loaded straight into LDS (global_load_lds) when K % 64 == 0; the large
//            tiles' waves work as two groups out of step.
// Both need K % 8 == 0 and 16-byte aligned rows (16-byte loads); otherwise the
// caller falls back to the plain kernel.
//
// The order in which an output's products are summed depends on K, N and the
// kernel, never on M, the row's place in the batch or the tile it falls in.
// Replaces the reference's matvec_bf16_simd / gemm_bf16 (shaders/ops.metal:52-159,
// :1090-1143); unlike gemm_bf16 (:1107) the accumulator is 32-bit.
#include "cache_layout.h"
#include "gemm.h"

#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *(const bf16x8*)p; }
__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16)0.0f;
    return z;
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
// The value the neighbouring lane (lane ^ 1) passes: a DPP move within each group of four lanes, no LDS.
__device__ __forceinline__ float swap_neighbours(float x) {
    int u = __float_as_int(x);
    return __int_as_float(__builtin_amdgcn_update_dpp(u, u, 0xB1, 0xf, 0xf, true));     // quad_perm [1, 0, 3, 2]
}
// x / (1 + exp(-x)) with the device's exponential and reciprocal instructions (each within an ulp; the result is
// rounded to bfloat16 right after).  For the epilogues that finish thousands of values per wave.
__device__ __forceinline__ float silu_fast_f32(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896341f));
}

// The tile loops' barrier: this wave's LDS reads and writes are done, then every wave of the block
// has arrived.  Unlike __syncthreads() it does not wait for loads from memory that are still in
// flight (the later tiles of a pipeline); the "memory" clobber keeps the compiler from moving
// memory accesses across it.
__device__ __forceinline__ void block_sync_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

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
// With gridDim.y > 1 the k-blocks are shared out over that many blocks as well
// (contiguous ranges): each writes its 32-bit partial sums to `partial`
// [gridDim.y][M][N] and gemm_splitk_finish_kernel adds them in order and applies
// the epilogue.  That is for weights with few rows and many tokens (17..64),
// where blocks of 64 features are needed to keep the tokens' rows from being
// read too often, and would otherwise be too few to fill the device.
// ---------------------------------------------------------------------------
// LAST < 16: the last of a block's feature tiles has only LAST features (a block of 24 features is a tile and a
// half): the rows beyond are never asked for (their lanes load nothing and multiply zeros), so a weight whose
// 16-feature blocks would be one and a half rounds of the device can be shared out evenly.
template <int MT, int NT, int NW, int U, int LAST = 16>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ A, int lda,
                                                              const bf16* __restrict__ W, void* __restrict__ out,
                                                              int ldc, int M, int N, int K, int epi,
                                                              float* __restrict__ partial, QkvEpilogue qe, int rot_feats,
                                                              RowScale rs, NextNorm nn) {
    extern __shared__ __attribute__((aligned(16))) unsigned char skinny_smem[];
    float* red = (float*)skinny_smem;          // [NW][MT][NT][4][64]
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int row = lane & 15, g = lane >> 4;
    constexpr int BF = (NT - 1) * 16 + LAST;       // features of a block
    static_assert(LAST == 16 || LAST == 8, "a whole last tile, or half of one");
    int n0 = blockIdx.x * BF;
    const bool last_asks = LAST == 16 || row < LAST;   // whether this lane's row of the last tile exists
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
    int nkb = (K + 63) / 64;
    int per = (nkb + gridDim.y - 1) / gridDim.y;
    int lo = blockIdx.y * per;
    int kb_hi = min(nkb, lo + per);                        // this block's k-blocks: [lo, kb_hi)
    int cnt = max(min(full, kb_hi) - lo, 0);               // the full ones among them
    // The block walks its full k-blocks starting at `rot` and wraps round: with rot_feats > 0,
    // neighbouring groups of rot_feats features are at different places of their rows at any
    // moment.  Rows are a multiple of the memory channels' interleave apart, so blocks in step
    // would all ask the same few channels at once.  The start depends on the features alone
    // (a block's features lie within one group), not on how many of them a block takes.
    int rot = (cnt > 0 && rot_feats > 0) ? (n0 / rot_feats) % cnt : 0;
    auto turn = [&](int j) { int x = j + rot; return lo + (x >= cnt ? x - cnt : x); };
    // out += sum: the old values of the tile this wave will finish are asked for now, so that
    // their trip to memory runs beside the weights' instead of after the sums are ready
    float old[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float next_w[4] = {0.0f, 0.0f, 0.0f, 0.0f};     // the next norm's weight for the same features, if something is left for it
    const bool old_ahead = epi == LLMRS_EPI_ACCUM_F32 && partial == nullptr && wave < MT * NT;
    if (old_ahead) {
        int m = (wave / NT) * 16 + row, n = n0 + (wave % NT) * 16 + 4 * g;
        if (m < M)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) {
                    old[r] = ((const float*)out)[(size_t)m * ldc + n + r];
                    if (nn.sumsq != nullptr) next_w[r] = nn.weight[n + r];
                }
    }
    int j = wave;
    for (; j + (U - 1) * NW < cnt; j += U * NW) {
        bf16x8 w[U][NT][2], x[U][MT][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int k = turn(j + u * NW) * 64 + g * 8;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (LAST == 16 || nt < NT - 1 || last_asks) { w[u][nt][0] = load8(wp[nt] + k); w[u][nt][1] = load8(wp[nt] + k + 32); }
                else { w[u][nt][0] = zero8(); w[u][nt][1] = zero8(); }
            }
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
    // what is left of this wave's turns, then the partial block if it is the wave's turn
    for (;; j += NW) {
        bool partial_turn = j == cnt && kb_hi > lo + cnt;   // one k-block past the full ones, cut by K
        if (j >= cnt && !partial_turn) break;
        int k = (partial_turn ? lo + cnt : turn(j)) * 64 + g * 8;
        bool v0 = k < K, v1 = k + 32 < K;
        bf16x8 w0[NT], w1[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            bool asks = LAST == 16 || nt < NT - 1 || last_asks;
            w0[nt] = v0 && asks ? load8(wp[nt] + k) : zero8();
            w1[nt] = v1 && asks ? load8(wp[nt] + k + 32) : zero8();
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
        if (partial_turn) break;
    }
    // A norm left to this product (RowScale, up to 16 rows, so MT = 1): the waves that will finish tiles find their
    // row's scale now, so that the trip for the partial sums of squares runs beside the other waves' last rounds and
    // the barrier.  The row's four lanes take every fourth group of four parts in ascending order and add their sums
    // pairwise; every lane of a row, in every block, ends with the same bits.
    float inv_row = 1.0f;
    if (rs.sumsq != nullptr && wave < MT * NT) {
        const float* sp = rs.sumsq + (size_t)min(row, M - 1) * rs.nparts;
        float ss = 0.0f;
        if (rs.nparts % 16 == 0 && ((uintptr_t)rs.sumsq & 15) == 0) {
            // up to sixteen loads on their way at a time (the sums were written on other XCDs and come from memory);
            // a group past the row's parts adds zeros
            for (int base = 4 * g; base < rs.nparts; base += 256) {
                f32x4 p[16];
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    p[t] = base + 16 * t < rs.nparts ? *(const f32x4*)(sp + base + 16 * t) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 16; ++t) { ss += p[t][0]; ss += p[t][1]; ss += p[t][2]; ss += p[t][3]; }
            }
        } else {
            for (int i = 4 * g; i < rs.nparts; i += 16)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (i + q < rs.nparts) ss += sp[i + q];
        }
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        inv_row = 1.0f / sqrtf(ss / (float)K + rs.eps);
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
            v[r] = s * inv_row;      // (1 without a norm left to this product; with one, MT = 1 and the lane's row is `row`)
        }
        int m = mt * 16 + row;
        int n = n0 + nt * 16 + 4 * g;
        if (m >= M) continue;
        if (LAST < 16 && nt == NT - 1 && 4 * g >= LAST) continue;     // the half of the last tile that is the next block's
        if (partial != nullptr) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) partial[((size_t)blockIdx.y * M + m) * N + n + r] = v[r];
        } else if (epi == LLMRS_EPI_SWIGLU) {
#pragma unroll
            for (int r = 0; r < 4; r += 2)
                if (n + r + 1 < N) ((bf16*)out)[(size_t)m * ldc + (n + r) / 2] = (bf16)(silu_f32(v[r]) * v[r + 1]);
        } else if (epi == LLMRS_EPI_QKV) {
            // four consecutive features of one head: two rotation pairs (2i, 2i+1); the
            // rotation is applied to the 32-bit sums, which are rounded once
            if (n >= N) continue;
            int hd = qe.head_dim, head = n / hd, d = n % hd;
            bool is_q = head < qe.n_heads, is_k = !is_q && head < qe.n_heads + qe.n_kv_heads;
            if (is_q || is_k) {
                float pos = (float)qe.positions[m];
#pragma unroll
                for (int r = 0; r < 4; r += 2)
                    if (d + r < qe.rotary_dim) {
                        float sn, cs;
                        sincosf(pos * qe.inv_freq[(d + r) >> 1], &sn, &cs);
                        float a = v[r], b = v[r + 1];
                        v[r] = a * cs - b * sn;
                        v[r + 1] = a * sn + b * cs;
                    }
            }
            bf16x4 o4;
#pragma unroll
            for (int r = 0; r < 4; ++r) o4[r] = (bf16)v[r];
            if (is_q) {
                *(bf16x4*)((bf16*)out + (size_t)m * ldc + n) = o4;
            } else if (qe.write_kv) {
                int slot = qe.slot_map[m];
                if (slot < 0 || slot >= qe.num_pages * qe.page_size) continue;   // never write outside the cache
                int page = slot / qe.page_size, off = slot % qe.page_size;
                if (is_k) {
                    int kvh = head - qe.n_heads;
                    *(bf16x4*)(qe.k_cache + k_cache_index(page, kvh, off, d, qe.n_kv_heads, qe.page_size, hd)) = o4;
                } else {
                    int kvh = head - qe.n_heads - qe.n_kv_heads;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        qe.v_cache[v_cache_index(page, kvh, off, d + r, qe.n_kv_heads, qe.page_size, hd)] = o4[r];
                }
            }
        } else if (old_ahead && tile == wave) {
            float ss = 0.0f;
            bf16x4 y4;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float nv = 0.0f;
                if (n + r < N) {
                    nv = old[r] + v[r];
                    ((float*)out)[(size_t)m * ldc + n + r] = nv;
                    ss = fmaf(nv, nv, ss);
                    nv *= next_w[r];
                }
                y4[r] = (bf16)nv;
            }
            if (nn.sumsq != nullptr) {
                // for the norm that follows (NextNorm).  The row's four lanes hold four features each of this tile's
                // sixteen; they are all here: a row is in the batch for all of them or for none.
                if (n + 3 < N) *(bf16x4*)(nn.y + (size_t)m * nn.ldy + n) = y4;
                else
                    for (int r = 0; r < 4; ++r)
                        if (n + r < N) nn.y[(size_t)m * nn.ldy + n + r] = y4[r];
                ss += __shfl_xor(ss, 16, 64);
                if constexpr (LAST == 16) {
                    ss += __shfl_xor(ss, 32, 64);
                    if (g == 0) nn.sumsq[(size_t)m * ((N + 15) / 16) + (n0 / 16 + nt)] = ss;
                } else {
                    // blocks of 8 features (NT = 1: the launcher sees to it): a part is the block's 8, held by two lanes
                    if (g == 0) nn.sumsq[(size_t)m * ((N + 7) / 8) + n0 / 8] = ss;
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) epilogue_store<bf16>(epi, out, ldc, m, n + r, v[r]);
        }
    }
}

// Adds the partial sums of a split product in order and applies the epilogue.
// One thread for two adjacent features (a gate/up pair when the epilogue is SwiGLU).
__global__ void gemm_splitk_finish_kernel(const float* __restrict__ partial, int splits, void* __restrict__ out,
                                          int ldc, int M, int N, int epi) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t pairs = (size_t)M * ((N + 1) / 2);
    if (idx >= pairs) return;
    int m = (int)(idx / ((N + 1) / 2)), n = 2 * (int)(idx % ((N + 1) / 2));
    float v0 = 0.0f, v1 = 0.0f;
    bool has1 = n + 1 < N;
    for (int s = 0; s < splits; ++s) {
        const float* p = partial + ((size_t)s * M + m) * N + n;
        v0 += p[0];
        if (has1) v1 += p[1];
    }
    if (epi == LLMRS_EPI_SWIGLU) {
        if (has1) ((bf16*)out)[(size_t)m * ldc + n / 2] = (bf16)(silu_f32(v0) * v1);
    } else {
        epilogue_store<bf16>(epi, out, ldc, m, n, v0);
        if (has1) epilogue_store<bf16>(epi, out, ldc, m, n + 1, v1);
    }
}

// The same for a product that adds into the 32-bit stream and is followed by a norm x / rms(x) * weight: a block
// for each row adds the parts in the same order, writes the stream's new row, and, having the whole row, the
// normed row as well (NextNorm with eps): no norm kernel runs.  Up to 16384 features (16 per thread), a multiple of 4.
__global__ __launch_bounds__(1024) void gemm_splitk_finish_norm_kernel(const float* __restrict__ partial, int splits,
                                                                        float* __restrict__ out, int ldc, int M, int N,
                                                                        NextNorm nn) {
    __shared__ float red[16];
    int m = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const float* p0 = partial + (size_t)m * N;
    float* o = out + (size_t)m * ldc;
    f32x4 h[4];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int n = (i * (int)blockDim.x + tid) * 4;
        h[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (n < N) {
            f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int s = 0; s < splits; ++s) v += *(const f32x4*)(p0 + (size_t)s * M * N + n);
            h[i] = *(const f32x4*)(o + n) + v;
            *(f32x4*)(o + n) = h[i];
#pragma unroll
            for (int r = 0; r < 4; ++r) ss = fmaf(h[i][r], h[i][r], ss);
        }
    }
    ss = wave_sum(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < waves; ++w) total += red[w];
    float inv = 1.0f / sqrtf(total / (float)N + nn.eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int n = (i * (int)blockDim.x + tid) * 4;
        if (n < N) {
            f32x4 w = *(const f32x4*)(nn.weight + n);
            bf16x4 y;
#pragma unroll
            for (int r = 0; r < 4; ++r) y[r] = (bf16)(h[i][r] * inv * w[r]);
            *(bf16x4*)(nn.y + (size_t)m * nn.ldy + n) = y;
        }
    }
}
// Adds the parts of a split product up: with the norm that follows where one is to be finished (NextNorm with eps).
static void launch_splitk_finish(hipStream_t stream, const float* partial, int splits, void* out, int ldc, int M, int N,
                                 int epi, const NextNorm* next) {
    if (next != nullptr && next->eps > 0.0f) {
        int threads = min(1024, ceil_div(ceil_div(N, 4), 64) * 64);
        gemm_splitk_finish_norm_kernel<<<M, threads, 0, stream>>>(partial, splits, (float*)out, ldc, M, N, *next);
        return;
    }
    size_t pairs = (size_t)M * ((N + 1) / 2);
    gemm_splitk_finish_kernel<<<ceil_div(pairs, 256), 256, 0, stream>>>(partial, splits, out, ldc, M, N, epi);
}

template <int MT, int NT, int NW, int U, int LAST = 16>
static void launch_skinny(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                          int M, int N, int K, int epi, const QkvEpilogue* qkv, int splits = 1,
                          float* partial = nullptr, int rot_feats = 0, const RowScale* scale = nullptr,
                          const NextNorm* next = nullptr) {
    size_t bytes = (size_t)NW * MT * NT * 4 * 64 * sizeof(float);
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, NT, NW, U, LAST>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        configured = true;
    }
    dim3 grid(ceil_div(N, (NT - 1) * 16 + LAST), splits);
    gemm_skinny_kernel<MT, NT, NW, U, LAST><<<grid, NW * 64, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi,
                                                                          splits > 1 ? partial : nullptr,
                                                                          qkv ? *qkv : QkvEpilogue{}, rot_feats,
                                                                          scale ? *scale : RowScale{},
                                                                          next && splits == 1 ? *next : NextNorm{});
    if (splits > 1) launch_splitk_finish(stream, partial, splits, out, ldc, M, N, epi, next);
}

// ---------------------------------------------------------------------------
// tiled: C[m, n] = sum_k X[m, k] W[n, k]
//   A operand = X rows (lane l: row l%32, k-chunk l/32), B operand = W rows
//   C: lane l holds feature l%32 and tokens 8*(r/4) + 4*(l/32) + r%4, r = 0..15,
//   so a store instruction writes 32 consecutive features of a token.
// ---------------------------------------------------------------------------
// BM x BN output tile per block of four waves (2 x 2); K in steps of BKT through
// two LDS buffers.  The global loads of the next P tiles are in flight, in
// registers, while this one is multiplied (one tile's product is far shorter than
// a trip to memory); the oldest of them is written to the other LDS buffer
// before the step's one barrier.
// LDS rows are padded by 16 bytes so that 16 lanes' 16-byte reads hit distinct banks.
template <int BM, int BN, int BKT, int P>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ A, int lda,
                                                         const bf16* __restrict__ W, void* __restrict__ out,
                                                         int ldc, int M, int N, int K, int epi) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    bf16* smem = (bf16*)smem_raw;
    constexpr int LDT = BKT + 8;
    constexpr int TM = BM / 2, TN = BN / 2, FM = TM / 32, FN = TN / 32;
    constexpr int TPR = BKT / 8;              // threads that stage one row (16 bytes each)
    constexpr int RPP = 256 / TPR;            // rows staged per pass
    constexpr int A_IT = BM / RPP, W_IT = BN / RPP, BUF = (BM + BN) * LDT;
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave >> 1, wn = wave & 1;
    int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int srow = tid / TPR, schunk = (tid % TPR) * 8;
    bf16x8 ra[P][A_IT], rw[P][W_IT];     // ring of tiles in flight: slot t % P holds tile t

    auto load_tile = [&](int kt, int slot) {
        int k = kt * BKT + schunk;
        bool in = k < K;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) {
            int gm = min(m0 + srow + RPP * i, M - 1);
            ra[slot][i] = in ? load8(A + (size_t)gm * lda + k) : zero8();
        }
#pragma unroll
        for (int i = 0; i < W_IT; ++i) {
            int gn = min(n0 + srow + RPP * i, N - 1);
            rw[slot][i] = in ? load8(W + (size_t)gn * K + k) : zero8();
        }
    };
    auto store_tile = [&](int buf, int slot) {
        bf16* as = smem + buf * BUF;
        bf16* ws = as + BM * LDT;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) *(bf16x8*)(as + (srow + RPP * i) * LDT + schunk) = ra[slot][i];
#pragma unroll
        for (int i = 0; i < W_IT; ++i) *(bf16x8*)(ws + (srow + RPP * i) * LDT + schunk) = rw[slot][i];
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    int nk = (K + BKT - 1) / BKT;
    load_tile(0, 0);
    store_tile(0, 0);
#pragma unroll
    for (int p = 1; p <= P - 1; ++p)
        if (p < nk) load_tile(p, p % P);
    __syncthreads();
    int frow = lane & 31, fk = (lane >> 5) * 8;
    for (int kt0 = 0; kt0 < nk; kt0 += P) {
#pragma unroll
        for (int p = 0; p < P; ++p) {            // unrolled so that ring slots are compile-time
            int kt = kt0 + p;
            if (kt >= nk) break;
            int cur = kt & 1;
            // tile kt's slot (p) is free: tile kt went to LDS in the step before
            if (kt + P < nk) load_tile(kt + P, p);
            const bf16* as = smem + cur * BUF + (wm * TM + frow) * LDT + fk;
            const bf16* ws = smem + cur * BUF + BM * LDT + (wn * TN + frow) * LDT + fk;
#pragma unroll
            for (int ks = 0; ks < BKT / 16; ++ks) {
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
            if (kt + 1 < nk) store_tile(cur ^ 1, (p + 1) % P);
            // (a bare barrier: __syncthreads() would wait for the later tiles' loads as well)
            block_sync_lds();
        }
    }

    // The accumulators must be indexed by constants or they end up in scratch memory:
    // the tiles are walked by a compile-time loop.
    static_for<0, FM * FN>([&](auto idx) {
        constexpr int i = decltype(idx)::value / FN, j = decltype(idx)::value % FN;
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
    });
}

template <int BM, int BN, int BKT, int P>
static int launch_tiled(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                        int M, int N, int K, int epi) {
    static bool configured = false;
    size_t bytes = 2 * (BM + BN) * (BKT + 8) * sizeof(bf16);
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<BM, BN, BKT, P>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return llmrs_fail("gemm: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
        configured = true;
    }
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM));
    if (grid.y > 65535) return llmrs_fail("gemm: M=%d is too large for one launch", M);
    gemm_tiled_kernel<BM, BN, BKT, P><<<grid, 256, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
    return 0;
}

// What a block of the tiled kernels does with its sums.  `smem` is the block's LDS (SMEM_BYTES of
// it), free once every wave has left the tile loop.
template <int BM, int BN, int WGM, int WGN, int SMEM_BYTES>
__device__ __forceinline__ void tile_epilogue(f32x16 (&acc)[BM / WGM / 32][BN / WGN / 32], unsigned char* smem,
                                              void* __restrict__ out, int ldc, int M, int N, int epi,
                                              float* __restrict__ partial, int m0, int n0) {
    constexpr int WAVES = WGM * WGN;
    constexpr int TM = BM / WGM, TN = BN / WGN, FM = TM / 32, FN = TN / 32;
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int wm = wave / WGN, wn = wave % WGN;
    if (partial != nullptr) {       // one part of the sum: as it is, for the kernel that adds the parts
        float* part = partial + (size_t)blockIdx.z * M * N;
        static_for<0, FM * FN>([&](auto idx) {
            constexpr int i = decltype(idx)::value / FN, j = decltype(idx)::value % FN;
            int n = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < M && n < N) part[(size_t)m * N + n] = acc[i][j][r];
            }
        });
        return;
    }
    if (epi == LLMRS_EPI_ACCUM_F32) {
        // out += acc: a row block's old values are all asked for before the first sum is stored
        // (left to itself the compiler waits for each load before the store that follows it,
        // a trip to memory per value).
        float* o = (float*)out;
        static_for<0, FM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            float old[FN][16];
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                int n = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    old[j][r] = o[(size_t)min(m, M - 1) * ldc + min(n, N - 1)];
                }
            }
            static_for<0, FN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                int n = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < M && n < N) o[(size_t)m * ldc + n] = old[j][r] + acc[i][j][r];
                }
            });
        });
        return;
    }
    // 16-bit results: a lane holds one column of 16 rows, which stored as they lie would be 2 bytes
    // per lane and store.  The wave puts its tile through LDS (free after the loop's last barrier; each
    // wave has room for its own tile) and stores it row by row, 16 bytes per lane, whole lines at a time.
    bool staged = (epi == LLMRS_EPI_STORE || epi == LLMRS_EPI_SWIGLU) && ldc % 8 == 0 && ((uintptr_t)out & 15) == 0 &&
                  (epi == LLMRS_EPI_SWIGLU ? N % 16 == 0 : N % 8 == 0);
    if (staged) {
        const bool glu = epi == LLMRS_EPI_SWIGLU;
        const int cols = glu ? TN / 2 : TN;                       // columns of the wave's tile as stored
        const int row_bytes = cols * 2;
        static_assert(TN * 2 * TM * WAVES <= SMEM_BYTES, "the waves' tiles must fit in the tile buffers");
        unsigned char* mine = smem + wave * (TN * 2 * TM);
        // A lane holds one column of 16 rows, its neighbour (lane ^ 1) the next column.  Registers r and r + 1
        // are two adjacent rows: the two lanes trade one value of each pair (one DPP move, no LDS), after which the
        // even lane has both columns of row r and the odd lane both of row r + 1.  For the gate/up epilogue those
        // are a gate and its up (each lane finishes one output of the pair, none idles); for a plain store two
        // neighbouring results, written with one 4-byte store.
        const bool odd = lane & 1;
        static_for<0, FM * FN>([&](auto idx) {
            constexpr int i = decltype(idx)::value / FN, j = decltype(idx)::value % FN;
            int c = j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                int row = i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3) + (odd ? 1 : 0);
                float v0 = acc[i][j][r], v1 = acc[i][j][r + 1];
                float got = swap_neighbours(odd ? v0 : v1);
                float left = odd ? got : v0, right = odd ? v1 : got;       // columns c & ~1 and c | 1 of `row`
                if (glu) *(bf16*)(mine + row * row_bytes + (c / 2) * 2) = (bf16)(silu_fast_f32(left) * right);
                else {
                    bf16x2 two;
                    two[0] = (bf16)left;
                    two[1] = (bf16)right;
                    *(bf16x2*)(mine + row * row_bytes + (c & ~1) * 2) = two;
                }
            }
        });
        __builtin_amdgcn_s_waitcnt(0xc07f);                       // lgkmcnt(0): the wave's own LDS writes are done
        int lanes_per_row = cols / 8, rows_per_pass = 64 / lanes_per_row;
        int lr = lane / lanes_per_row, lc = (lane % lanes_per_row) * 8;
        int n_out = (glu ? (n0 + wn * TN) / 2 : n0 + wn * TN) + lc, n_lim = glu ? N / 2 : N;
        for (int row = lr; row < TM; row += rows_per_pass) {
            int m = m0 + wm * TM + row;
            if (m < M && n_out < n_lim)                           // (n_lim is a multiple of 8: a lane's 8 columns are in or out together)
                *(bf16x8*)((bf16*)out + (size_t)m * ldc + n_out) = *(const bf16x8*)(mine + row * row_bytes + lc * 2);
        }
        return;
    }
    static_for<0, FM * FN>([&](auto idx) {
        constexpr int i = decltype(idx)::value / FN, j = decltype(idx)::value % FN;
        int n = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            float v = acc[i][j][r];
            if (epi == LLMRS_EPI_SWIGLU) {
                float other = __shfl_xor(v, 1, 64);
                if (!(lane & 1) && m < M && n + 1 < N)
                    ((bf16*)out)[(size_t)m * ldc + n / 2] = (bf16)(silu_f32(v) * other);
            } else if (m < M && n < N) {
                epilogue_store<bf16>(epi, out, ldc, m, n, v);
            }
        }
    });
}

// ---------------------------------------------------------------------------
// tiled, loads straight into LDS: for K % 64 == 0.
// global_load_lds_dwordx4 moves 16 bytes per lane from memory into LDS without
// passing through registers; the 64 lanes of an instruction fill 1 KB of LDS in
// lane order, which is 8 tile rows of 64 k.  Rows therefore lie 128 bytes apart,
// unpadded, and bank conflicts are avoided by a swizzle instead: the 16-byte
// chunk c of row r lies in slot c ^ ((r >> 1) & 7) of its row (each lane simply
// fetches the chunk that belongs in its slot), so the 16 lanes of an operand read,
// which want the same chunk of 16 consecutive rows, hit 16 different bank groups.
// STAGES tiles are in LDS; the loads of the tile STAGES-1 ahead are issued
// before this tile's products and waited for (s_waitcnt vmcnt) only as far as the
// next tile needs.  No staging registers, no LDS store instructions.
// ---------------------------------------------------------------------------
template <int N_>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N_ >= 0 && N_ < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N_ & 15) | (7 << 4) | (15 << 8) | ((N_ >> 4) << 14));
}

template <int BM, int BN, int WGM, int WGN, int STAGES>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_dma_kernel(const bf16* __restrict__ A, int lda,
                                                       const bf16* __restrict__ W, void* __restrict__ out,
                                                       int ldc, int M, int N, int K, int epi,
                                                       float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char dma_smem[];
    constexpr int WAVES = WGM * WGN;                              // waves of a block, as a WGM x WGN grid over the tile
    constexpr int TM = BM / WGM, TN = BN / WGN, FM = TM / 32, FN = TN / 32;
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int A_GROUPS = BM / 8 / WAVES, W_GROUPS = BN / 8 / WAVES;   // 8-row groups per wave
    constexpr int LOADS = A_GROUPS + W_GROUPS;                     // load instructions per wave per tile
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave / WGN, wn = wave % WGN;
    int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int lrow = lane >> 3, lslot = lane & 7;

    // this lane's part of a tile: for each of its row groups, the row's global address of the
    // chunk that belongs in the lane's slot
    const bf16* ga[A_GROUPS];
    const bf16* gw[W_GROUPS];
#pragma unroll
    for (int i = 0; i < A_GROUPS; ++i) {
        int row = (wave * A_GROUPS + i) * 8 + lrow;
        ga[i] = A + (size_t)min(m0 + row, M - 1) * lda + ((lslot ^ ((row >> 1) & 7)) * 8);
    }
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) {
        int row = (wave * W_GROUPS + i) * 8 + lrow;
        gw[i] = W + (size_t)min(n0 + row, N - 1) * K + ((lslot ^ ((row >> 1) & 7)) * 8);
    }
    // With gridDim.z > 1 the k-tiles are shared out over that many blocks (contiguous ranges): each
    // writes its 32-bit sums to `partial` [gridDim.z][M][N] and gemm_splitk_finish_kernel adds them
    // in order and applies the epilogue.  That is for products with too few tiles to fill the device.
    int nk_all = K / 64, per_split = (nk_all + gridDim.z - 1) / gridDim.z;
    int kt_lo = blockIdx.z * per_split;
    int nk = max(0, min(nk_all, kt_lo + per_split) - kt_lo);       // this block's k-tiles: [kt_lo, kt_lo + nk)
    auto issue = [&](int kt, int stage) {
        kt += kt_lo;
        unsigned base = __builtin_amdgcn_readfirstlane(stage * STAGE_BYTES + wave * A_GROUPS * 1024);
#pragma unroll
        for (int i = 0; i < A_GROUPS; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ga[i] + kt * 64),
                                             (__attribute__((address_space(3))) void*)(dma_smem + base + i * 1024), 16, 0, 0);
        unsigned wbase = __builtin_amdgcn_readfirstlane(stage * STAGE_BYTES + BM * 128 + wave * W_GROUPS * 1024);
#pragma unroll
        for (int i = 0; i < W_GROUPS; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gw[i] + kt * 64),
                                             (__attribute__((address_space(3))) void*)(dma_smem + wbase + i * 1024), 16, 0, 0);
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if (p < nk) issue(p, p);
    if (nk >= STAGES - 1) wait_vmcnt<(STAGES - 2) * LOADS>(); else wait_vmcnt<0>();
    __syncthreads();

    int frow = lane & 31, h = lane >> 5;
    for (int kt = 0; kt < nk; ++kt) {
        int stage = kt % STAGES;
        if (kt + STAGES - 1 < nk) issue(kt + STAGES - 1, (kt + STAGES - 1) % STAGES);
        const unsigned char* as = dma_smem + stage * STAGE_BYTES;
        const unsigned char* ws = as + BM * 128;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            bf16x8 a[FM], b[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                int row = wm * TM + i * 32 + frow;
                a[i] = *(const bf16x8*)(as + row * 128 + (((ks * 2 + h) ^ ((row >> 1) & 7)) * 16));
            }
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                int row = wn * TN + j * 32 + frow;
                b[j] = *(const bf16x8*)(ws + row * 128 + (((ks * 2 + h) ^ ((row >> 1) & 7)) * 16));
            }
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        // the next tile must have landed before anybody reads it; later tiles may still be on their way
        // (a bare barrier: __syncthreads() would wait for every load in flight, the later tiles' too)
        if (kt + STAGES - 1 < nk) wait_vmcnt<(STAGES - 2) * LOADS>(); else wait_vmcnt<0>();
        block_sync_lds();
    }

    tile_epilogue<BM, BN, WGM, WGN, STAGES * STAGE_BYTES>(acc, dma_smem, out, ldc, M, N, epi, partial, m0, n0);
}

template <int BM, int BN, int WGM, int WGN, int STAGES>
static int launch_dma(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                      int M, int N, int K, int epi, int splits = 1, float* partial = nullptr, const NextNorm* next = nullptr,
                      bool finish = true) {
    static bool configured = false;
    size_t bytes = (size_t)STAGES * (BM + BN) * 128;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_dma_kernel<BM, BN, WGM, WGN, STAGES>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return llmrs_fail("gemm: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
        configured = true;
    }
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM), splits);
    if (grid.y > 65535) return llmrs_fail("gemm: M=%d is too large for one launch", M);
    gemm_dma_kernel<BM, BN, WGM, WGN, STAGES><<<grid, 64 * WGM * WGN, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi,
                                                                                      splits > 1 ? partial : nullptr);
    if (splits > 1 && finish) launch_splitk_finish(stream, partial, splits, out, ldc, M, N, epi, next);
    return 0;
}

// ---------------------------------------------------------------------------
// tiled, two groups of waves out of step: for K % 64 == 0, 256 x 256 tiles.
// In the tile loop above all eight waves of a block do the same thing at the same
// time: after each barrier every wave asks memory for the next tile, then reads LDS,
// then feeds the matrix cores, and the two waves that share a SIMD compete for each in
// turn.  Here the block's waves are two groups of four, one wave of each on every SIMD.
// A k-tile of 64 is four phases with a barrier after each: the operands of its first
// half from LDS into registers; their 16 MFMAs; the second half's operands; their
// MFMAs.  The second group runs one phase behind the first, so while one wave of a
// SIMD multiplies, the other reads LDS.  Both groups ask memory for the tile after the
// next in the same phase (the first group's first, the second group's fourth of the
// tile before), the first in which the buffer's last reader is done, and wait for it
// four phases later.  Every wave passes the same number of barriers.  Same LDS layout
// as above (two tiles, rows of 128 bytes, chunks swizzled), same order of sums: the
// results are bitwise those of the loop above.  A wave multiplies at raised priority.
// (Measured on MI355X, 2048 x 4096 times 24576 features: 2-5 % faster than the loop above when
// the product runs back to back with itself, 1 % inside a prompt step of the 8B shape.)
// ---------------------------------------------------------------------------
template <int BM, int BN, int WGM, int WGN, bool BUF = false>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_pingpong_kernel(const bf16* __restrict__ A, int lda,
                                                            const bf16* __restrict__ W, void* __restrict__ out,
                                                            int ldc, int M, int N, int K, int epi) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char pp_smem[];
    constexpr int WAVES = WGM * WGN;
    static_assert(WAVES == 8, "two groups of four waves");
    constexpr int TM = BM / WGM, TN = BN / WGN, FM = TM / 32, FN = TN / 32;
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int A_GROUPS = BM / 8 / WAVES, W_GROUPS = BN / 8 / WAVES;   // 8-row groups per wave
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave / WGN, wn = wave % WGN;
    int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int lrow = lane >> 3, lslot = lane & 7;
    const bf16* ga[A_GROUPS];
    const bf16* gw[W_GROUPS];
#pragma unroll
    for (int i = 0; i < A_GROUPS; ++i) {
        int row = (wave * A_GROUPS + i) * 8 + lrow;
        ga[i] = A + (size_t)min(m0 + row, M - 1) * lda + ((lslot ^ ((row >> 1) & 7)) * 8);
    }
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) {
        int row = (wave * W_GROUPS + i) * 8 + lrow;
        gw[i] = W + (size_t)min(n0 + row, N - 1) * K + ((lslot ^ ((row >> 1) & 7)) * 8);
    }
    const int nk = K / 64;
    // BUF: the loads go through buffer descriptors (a scalar base and a 32-bit offset per lane)
    // instead of a 64-bit address per lane; the caller sees to it that both operands are under 4 GB.
    // (The descriptor type and builtins exist for the device only.)
#if defined(__HIP_DEVICE_COMPILE__)
    __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)min((size_t)M * lda * 2, (size_t)0xffffffffu), 0x00020000);
    __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)min((size_t)N * K * 2, (size_t)0xffffffffu), 0x00020000);
#endif
    unsigned oa[A_GROUPS], ow[W_GROUPS];
#pragma unroll
    for (int i = 0; i < A_GROUPS; ++i) oa[i] = (unsigned)((const char*)ga[i] - (const char*)A);
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) ow[i] = (unsigned)((const char*)gw[i] - (const char*)W);
    auto issue = [&](int kt) {
        if (kt >= nk) return;
        int stage = kt & 1;
        unsigned base = __builtin_amdgcn_readfirstlane(stage * STAGE_BYTES + wave * A_GROUPS * 1024);
#pragma unroll
        for (int i = 0; i < A_GROUPS; ++i) {
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr (BUF)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (__attribute__((address_space(3))) void*)(pp_smem + base + i * 1024), 16, oa[i], kt * 128, 0, 0);
            else
#endif
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ga[i] + kt * 64),
                                                 (__attribute__((address_space(3))) void*)(pp_smem + base + i * 1024), 16, 0, 0);
        }
        unsigned wbase = __builtin_amdgcn_readfirstlane(stage * STAGE_BYTES + BM * 128 + wave * W_GROUPS * 1024);
#pragma unroll
        for (int i = 0; i < W_GROUPS; ++i) {
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr (BUF)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (__attribute__((address_space(3))) void*)(pp_smem + wbase + i * 1024), 16, ow[i], kt * 128, 0, 0);
            else
#endif
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gw[i] + kt * 64),
                                                 (__attribute__((address_space(3))) void*)(pp_smem + wbase + i * 1024), 16, 0, 0);
        }
    };
    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto barrier = [] {
        __builtin_amdgcn_sched_barrier(0);
        block_sync_lds();
        __builtin_amdgcn_sched_barrier(0);
    };
    auto lds_done = [] { __builtin_amdgcn_s_waitcnt(0xc07f); };     // lgkmcnt(0)
    int frow = lane & 31, h = lane >> 5;
    bf16x8 a[2][FM], b[2][FN];
    auto read_half = [&](int kt, int half) {
        const unsigned char* as = pp_smem + (kt & 1) * STAGE_BYTES;
        const unsigned char* ws = as + BM * 128;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            int ks = half * 2 + s2;
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                int row = wm * TM + i * 32 + frow;
                a[s2][i] = *(const bf16x8*)(as + row * 128 + (((ks * 2 + h) ^ ((row >> 1) & 7)) * 16));
            }
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                int row = wn * TN + j * 32 + frow;
                b[s2][j] = *(const bf16x8*)(ws + row * 128 + (((ks * 2 + h) ^ ((row >> 1) & 7)) * 16));
            }
        }
    };
    auto multiply = [&] {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s2][i], b[s2][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
    };

    issue(0);
    wait_vmcnt<0>();
    barrier();
    const int grp = wave >> 2;
    // Phases as the whole block sees them, p = 0, 1, ...: the first group works on k-tile kt in
    // phases 4 kt .. 4 kt + 3, the second in 4 kt + 1 .. 4 kt + 4.  Tile kt + 1 goes into the buffer
    // of tile kt - 1, whose last reader (the second group's third phase) is done when phase 4 kt
    // begins; it is first read in phase 4 kt + 4.
    if (grp == 1) { issue(1); barrier(); }
    for (int kt = 0; kt < nk; ++kt) {
        read_half(kt, 0);
        if (grp == 0) issue(kt + 1);                     // phase 4 kt: the buffer of tile kt - 1 is free
        lds_done();
        barrier();
        multiply();
        barrier();
        read_half(kt, 1);
        lds_done();
        if (grp == 1) wait_vmcnt<0>();                   // its part of tile kt + 1 (asked for four phases ago)
        barrier();
        if (grp == 1) issue(kt + 2);                     // phase 4 kt + 4: the buffer of tile kt is free
        multiply();
        if (grp == 0) wait_vmcnt<0>();
        barrier();
    }
    if (grp == 0) barrier();
    tile_epilogue<BM, BN, WGM, WGN, 2 * STAGE_BYTES>(acc, pp_smem, out, ldc, M, N, epi, nullptr, m0, n0);
}

template <int BM, int BN, int WGM, int WGN, bool BUF = false>
static int launch_pingpong(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                           int M, int N, int K, int epi) {
    static bool configured = false;
    size_t bytes = (size_t)2 * (BM + BN) * 128;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_pingpong_kernel<BM, BN, WGM, WGN, BUF>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return llmrs_fail("gemm: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
        configured = true;
    }
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM));
    if (grid.y > 65535) return llmrs_fail("gemm: M=%d is too large for one launch", M);
    gemm_pingpong_kernel<BM, BN, WGM, WGN, BUF><<<grid, 64 * WGM * WGN, bytes, stream>>>(A, lda, W, out, ldc, M, N, K, epi);
    return 0;
}

// ---------------------------------------------------------------------------
// tiled, four waves: for K % 64 == 0, tiles of 256 x 256.
// One wave per SIMD with a tile of 128 x 128 outputs, all of them in the accumulation registers (256 of them):
// a third fewer LDS reads per MFMA than the eight-wave tiles, and nothing shares the SIMD with the wave, so the
// loop is written so that the wave itself always has work in flight.  A k-tile of 64 is four steps of 16; each
// step asks LDS for the operands of the next step, moves a quarter of the next k-tile from registers into the
// other LDS buffer, asks memory for the same quarter of the k-tile after that, and multiplies the operands the
// step before it asked for.  Loads from memory pass through registers here, two k-tiles ahead of their use (the
// loads straight into LDS of the loops above hold a wave that has no partner on its SIMD up while the memory
// pipeline takes them).  The barrier between k-tiles stands before the last step's products, which run on
// registers read before it: the matrix cores work across the barrier.  Same LDS layout and order of sums as the
// loops above: bitwise the same results.  The epilogue is a template argument: with all of them in one kernel the
// compiler keeps a tile's 256 sums and every epilogue's temporaries alive together and spills.
// (Measured on MI355X, 2048 x 4096 times 24576 features with the gate/up epilogue, inside a prompt step of the 8B
// shape: 356 us against 372-376 for the eight waves in two groups and 367 with loads straight into LDS.)
// ---------------------------------------------------------------------------
// What a wave of the four-wave tile does with its sums: one band of 32 rows at a time.  16-bit results go through
// the wave's own part of LDS and leave as whole rows of the band, 16 bytes a lane; the 32-bit epilogues read and
// write memory directly (a lane half holds 32 consecutive columns of a row: whole lines).
template <int BM, int BN, int EPI>
__device__ __forceinline__ void band_epilogue(f32x16 (&acc)[BM / 64][BN / 64], unsigned char* smem, void* __restrict__ out,
                                              int ldc, int M, int N, int m0, int n0) {
    constexpr int TM = BM / 2, TN = BN / 2, FM = TM / 32, FN = TN / 32;
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int wm = wave / 2, wn = wave % 2;
    int c = lane & 31, hh = lane >> 5;
    if constexpr (EPI == LLMRS_EPI_ACCUM_F32 || EPI == LLMRS_EPI_STORE_F32) {
        float* o = (float*)out;
        static_for<0, FM * FN>([&](auto idx) {
            constexpr int i = decltype(idx)::value / FN, j = decltype(idx)::value % FN;
            int n = n0 + wn * TN + j * 32 + c;
            float old[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
                old[r] = EPI == LLMRS_EPI_ACCUM_F32 ? o[(size_t)min(m, M - 1) * ldc + min(n, N - 1)] : 0.0f;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int m = m0 + wm * TM + i * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
                if (m < M && n < N) o[(size_t)m * ldc + n] = old[r] + acc[i][j][r];
            }
            __builtin_amdgcn_sched_barrier(0);       // one part of the tile at a time: its old values are not asked for earlier
        });
    } else {
        constexpr bool glu = EPI == LLMRS_EPI_SWIGLU;
        constexpr int cols = glu ? TN / 2 : TN;      // columns of the wave's band as stored
        constexpr int row_bytes = cols * 2;
        unsigned char* mine = smem + wave * (32 * TN * 2);
        constexpr int pieces_per_row = cols / 8;     // 16-byte pieces in a row of the band
        int n_first = glu ? (n0 + wn * TN) / 2 : n0 + wn * TN, n_lim = glu ? N / 2 : N;
        const bool odd = lane & 1;
        static_for<0, FM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<0, FN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                int cc = j * 32 + c;
#pragma unroll
                for (int r = 0; r < 16; r += 2) {                 // (pairs of lanes trade values as in tile_epilogue)
                    int row = 8 * (r >> 2) + 4 * hh + (r & 3) + (odd ? 1 : 0);
                    float v0 = acc[i][j][r], v1 = acc[i][j][r + 1];
                    float got = swap_neighbours(odd ? v0 : v1);
                    float left = odd ? got : v0, right = odd ? v1 : got;
                    if (glu) *(bf16*)(mine + row * row_bytes + (cc / 2) * 2) = (bf16)(silu_fast_f32(left) * right);
                    else {
                        bf16x2 two;
                        two[0] = (bf16)left;
                        two[1] = (bf16)right;
                        *(bf16x2*)(mine + row * row_bytes + (cc & ~1) * 2) = two;
                    }
                }
            });
            __builtin_amdgcn_s_waitcnt(0xc07f);                   // lgkmcnt(0): the wave's own LDS writes are done
            for (int piece = lane; piece < 32 * pieces_per_row; piece += 64) {
                int row = piece / pieces_per_row, lc = (piece % pieces_per_row) * 8;
                int m = m0 + wm * TM + i * 32 + row;
                if (m < M && n_first + lc < n_lim)                // (n_lim is a multiple of 8: a lane's 8 columns are in or out together)
                    *(bf16x8*)((bf16*)out + (size_t)m * ldc + n_first + lc) = *(const bf16x8*)(mine + row * row_bytes + lc * 2);
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);                   // the band's rows are read before the next band overwrites them
            __builtin_amdgcn_sched_barrier(0);
        });
    }
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int BM, int BN, int EPI>
__global__ __launch_bounds__(256) void gemm_fourwave_kernel(const bf16* __restrict__ A, int lda, const bf16* __restrict__ W,
                                                            void* __restrict__ out, int ldc, int M, int N, int K) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char fw_smem[];
    constexpr int WAVES = 4;
    constexpr int TM = BM / 2, TN = BN / 2, FM = TM / 32, FN = TN / 32;
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int A_GROUPS = BM / 8 / WAVES, W_GROUPS = BN / 8 / WAVES;   // 8-row groups per wave
    constexpr int QA = A_GROUPS / 4, QW = W_GROUPS / 4, QL = QA + QW;     // a quarter of a wave's loads of a k-tile
    static_assert(BM == 256 && BN % 64 == 0 && FM * FN <= 16, "a wave's sums fill at most the 256 accumulation registers");
    static_assert(A_GROUPS % 4 == 0 && W_GROUPS % 4 == 0, "a quarter of a k-tile's loads in each of its four steps");
    static_assert(32 * TN * 2 * WAVES <= 2 * STAGE_BYTES, "the waves' bands must fit in the tile buffers");
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave / 2, wn = wave % 2;
    int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int lrow = lane >> 3, lslot = lane & 7;
    // this lane's part of a tile: for each of its row groups, the byte offset of the chunk that belongs in the lane's
    // slot of the LDS image (the caller sees to it that both operands are under 4 GB: buffer descriptors)
    unsigned oa[A_GROUPS], ow[W_GROUPS];
#pragma unroll
    for (int i = 0; i < A_GROUPS; ++i) {
        int row = (wave * A_GROUPS + i) * 8 + lrow;
        oa[i] = (unsigned)(((size_t)min(m0 + row, M - 1) * lda + ((lslot ^ ((row >> 1) & 7)) * 8)) * 2);
    }
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) {
        int row = (wave * W_GROUPS + i) * 8 + lrow;
        ow[i] = (unsigned)(((size_t)min(n0 + row, N - 1) * K + ((lslot ^ ((row >> 1) & 7)) * 8)) * 2);
    }
    const int nk = K / 64;
#if defined(__HIP_DEVICE_COMPILE__)
    __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)min((size_t)M * lda * 2, (size_t)0xffffffffu), 0x00020000);
    __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)min((size_t)N * K * 2, (size_t)0xffffffffu), 0x00020000);
#endif
    u32x4 sa[A_GROUPS], sw_[W_GROUPS];          // the k-tile on its way, in registers
    // quarter q of this wave's loads of k-tile kt, into registers (past the end: the last tile once more, never used)
    auto ask = [&](int kt, auto qc) {
        constexpr int q = decltype(qc)::value;
        kt = min(kt, nk - 1);
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int i = q * QA; i < (q + 1) * QA; ++i) sa[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, oa[i], kt * 128, 0);
#pragma unroll
        for (int i = q * QW; i < (q + 1) * QW; ++i) sw_[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, ow[i], kt * 128, 0);
#endif
    };
    // quarter q of the registers into the LDS buffer of k-tile kt: a load's 64 lanes fill 1 KB in lane order
    auto put = [&](int kt, auto qc) {
        constexpr int q = decltype(qc)::value;
        unsigned char* st = fw_smem + (kt & 1) * STAGE_BYTES;
#pragma unroll
        for (int i = q * QA; i < (q + 1) * QA; ++i) *(u32x4*)(st + (wave * A_GROUPS + i) * 1024 + lane * 16) = sa[i];
#pragma unroll
        for (int i = q * QW; i < (q + 1) * QW; ++i) *(u32x4*)(st + BM * 128 + (wave * W_GROUPS + i) * 1024 + lane * 16) = sw_[i];
    };
    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    int frow = lane & 31, h = lane >> 5;
    int sw = (frow >> 1) & 7;
    // LDS offsets of this lane's chunk for each of a tile's four k-steps (row tiles lie 4 KB apart)
    unsigned offa[4], offb[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        unsigned chunk = (unsigned)(((ks * 2 + h) ^ sw) * 16);
        offa[ks] = (wm * TM + frow) * 128 + chunk;
        offb[ks] = BM * 128 + (wn * TN + frow) * 128 + chunk;
    }
    bf16x8 fa[2][FM], fb[2][FN];
    auto read = [&](int kt, auto ksc, auto bufc) {
        constexpr int ks = decltype(ksc)::value, buf = decltype(bufc)::value;
        const unsigned char* st = fw_smem + (kt & 1) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[buf][i] = *(const bf16x8*)(st + offa[ks] + i * 32 * 128);
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[buf][j] = *(const bf16x8*)(st + offb[ks] + j * 32 * 128);
    };
    auto mult = [&](auto bufc) {
        constexpr int buf = decltype(bufc)::value;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][i], fb[buf][j], acc[i][j], 0, 0, 0);
    };
    // the order within a step: LDS reads, LDS writes and loads from memory each ahead of a group of the step's MFMAs
    auto order = [] {
        __builtin_amdgcn_sched_group_barrier(0x100, FM + FN, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x200, QL, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, QL, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, FM * FN - 8, 0);
    };
    // One step (a quarter of a k-tile).  While k-tile kt is multiplied, k-tile kt + 1 goes from registers into the
    // other LDS buffer and k-tile kt + 2 is asked for into the registers that frees.  A quarter written now was
    // asked for a k-tile ago; loads complete in order, so it is there when all but the three quarters asked for
    // since have completed.
    auto step = [&](int kt, auto ksc, auto qc, auto rbuf, auto mbuf, auto multiply) {
        read(kt, ksc, rbuf);
        wait_vmcnt<3 * QL>();
        put(kt + 1, qc);
        ask(kt + 2, qc);
        if constexpr (decltype(multiply)::value) mult(mbuf);
        order();
        __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    // k-tile 0 into LDS, k-tile 1 into registers
    ask(0, I0{}); ask(0, I1{}); ask(0, I2{}); ask(0, I3{});
    wait_vmcnt<0>();
    put(0, I0{}); put(0, I1{}); put(0, I2{}); put(0, I3{});
    ask(1, I0{}); ask(1, I1{}); ask(1, I2{}); ask(1, I3{});
    __syncthreads();               // (waits for the loads of k-tile 1 as well: once)
    // A step multiplies the operands that the step before it read; the last step's products of a k-tile run in the
    // first step of the next, on operands read before the barrier: the matrix cores work across it.
    auto k_tile = [&](int kt, auto not_first) {
        step(kt, I0{}, I0{}, I0{}, I1{}, not_first);
        step(kt, I1{}, I1{}, I1{}, I0{}, std::true_type{});
        step(kt, I2{}, I2{}, I0{}, I1{}, std::true_type{});
        step(kt, I3{}, I3{}, I1{}, I0{}, std::true_type{});
        block_sync_lds();          // this wave's LDS reads and writes are done, and everybody's
        __builtin_amdgcn_sched_barrier(0);
    };
    k_tile(0, std::false_type{});
    for (int kt = 1; kt < nk; ++kt) k_tile(kt, std::true_type{});
    mult(I1{});
    wait_vmcnt<0>();
    __syncthreads();
    band_epilogue<BM, BN, EPI>(acc, fw_smem, out, ldc, M, N, m0, n0);
}

// Whether the four-wave tiles can finish this product: the epilogues it has, 16-bit results as whole 16-byte pieces.
static bool fourwave_takes(int epi, const void* out, int ldc, int N) {
    if (epi == LLMRS_EPI_ACCUM_F32 || epi == LLMRS_EPI_STORE_F32) return true;
    if (epi == LLMRS_EPI_STORE) return ldc % 8 == 0 && ((uintptr_t)out & 15) == 0 && N % 8 == 0;
    if (epi == LLMRS_EPI_SWIGLU) return ldc % 8 == 0 && ((uintptr_t)out & 15) == 0 && N % 16 == 0;
    return false;
}
template <int BM, int BN, int EPI>
static int launch_fourwave_epi(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc, int M, int N, int K) {
    static bool configured = false;
    size_t bytes = (size_t)2 * (BM + BN) * 128;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_fourwave_kernel<BM, BN, EPI>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return llmrs_fail("gemm: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
        configured = true;
    }
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM));
    if (grid.y > 65535) return llmrs_fail("gemm: M=%d is too large for one launch", M);
    gemm_fourwave_kernel<BM, BN, EPI><<<grid, 256, bytes, stream>>>(A, lda, W, out, ldc, M, N, K);
    return 0;
}
// (operands under 4 GB each, K % 64 == 0, fourwave_takes(epi, ...): the caller's to check)
template <int BM, int BN>
static int launch_fourwave(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc, int M, int N, int K, int epi) {
    switch (epi) {
        case LLMRS_EPI_STORE: return launch_fourwave_epi<BM, BN, LLMRS_EPI_STORE>(stream, A, lda, W, out, ldc, M, N, K);
        case LLMRS_EPI_STORE_F32: return launch_fourwave_epi<BM, BN, LLMRS_EPI_STORE_F32>(stream, A, lda, W, out, ldc, M, N, K);
        case LLMRS_EPI_ACCUM_F32: return launch_fourwave_epi<BM, BN, LLMRS_EPI_ACCUM_F32>(stream, A, lda, W, out, ldc, M, N, K);
        case LLMRS_EPI_SWIGLU: return launch_fourwave_epi<BM, BN, LLMRS_EPI_SWIGLU>(stream, A, lda, W, out, ldc, M, N, K);
        default: return llmrs_fail("gemm: the four-wave tiles have no epilogue %d", epi);
    }
}

// Into how many parts the k range is split over blocks (1: not at all), by the product's shape alone.
// 17 to 64 rows (few-row kernel, 64 features per block): when the features give no more than 64
// blocks, until there are 256 of them, each part at least 16 k-blocks long (measured at 64 rows:
// 4096 x 14336 in 4 parts 35 us, in 8 parts 42; 2048 x 8192 in 8 parts 18 us, in 4 parts 23; at 32
// rows 4096 x 14336 40 -> 28 us, 2048 x 8192 24 -> 14; it no longer pays for N = 6144).
static int skinny_splits(int N, int K) {
    int blocks = ceil_div(N, 64), nkb = ceil_div(K, 64), splits = 1;
    while (blocks <= 64 && blocks * splits < 256 && splits < 16 && nkb / (splits * 2) >= 8) splits *= 2;
    return splits;
}
// Up to 256 rows whose 128 x 128 tiles are no more than the compute units: one block of eight waves per
// unit with four k-tiles in LDS (three on their way) instead of two blocks of four waves with two
// k-tiles each.  A tile's loads into LDS take longer than its MFMAs, and with few blocks per unit
// the deeper pipeline is what keeps them coming (measured, 128 rows at the 8B shapes: qkv 21.9 -> 19.7 us,
// o 21.3 -> 18.6, gate/up 76.6 -> 64.8, down 43.7 -> 36.6; 256 rows: o 25.8 -> 21.9, down 56.4 -> 50.9;
// with more tiles than units, or more rows, the two blocks win).
static bool deep_tiles(int M, int N, int K) {
    return K % 64 == 0 && M <= 256 && (long)ceil_div(M, 128) * ceil_div(N, 128) <= llmrs_compute_units();
}
// Above (128 x 128 tiles): until the tiles fill the places (two to a compute unit, or one where the
// deep pipeline runs), each part at least 8 k-tiles long.
static int tiled_splits(int M, int N, int K) {
    if (K % 64) return 1;
    long tiles = (long)ceil_div(M, 128) * ceil_div(N, 128);
    long places = (long)llmrs_compute_units() * (deep_tiles(M, N, K) ? 1 : 2);
    int nk = K / 64, splits = 1;
    while (tiles * splits * 2 <= places && splits < 16 && nk / (splits * 2) >= 8) splits *= 2;
    return splits;
}
// The 128 x 128 tiles of a product, in whichever of the two forms its shape asks for.
static int launch_tiles_128(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                            int M, int N, int K, int epi, int splits, float* partial, const NextNorm* next = nullptr,
                            bool finish = true) {
    if (deep_tiles(M, N, K)) return launch_dma<128, 128, 2, 4, 4>(stream, A, lda, W, out, ldc, M, N, K, epi, splits, partial, next, finish);
    return launch_dma<128, 128, 2, 2, 2>(stream, A, lda, W, out, ldc, M, N, K, epi, splits, partial, next, finish);
}
// 17..64 rows on a weight of middling width (more than 4096 features, fewer than the wide ones that
// get blocks of many feature tiles): the 128 x 128 tiles with k split over blocks read the tokens'
// rows less often than the few-row kernel's blocks of 32 features (measured at 64 rows:
// 10240 x 8192 90 -> 51 us, 8192 x 8192 49 -> 38, 8192 x 28672 160 -> 99, 6144 x 4096 31 -> 21;
// at 32 rows: 10240 x 8192 63 -> 48, 8192 x 28672 110 -> 90).
static bool few_rows_take_tiles(int M, int N, int K) {
    return M > 16 && M <= 64 && N > 4096 && N < 16384 && K % 64 == 0 && tiled_splits(M, N, K) > 1;
}
// Room (in floats) for the partial sums of a product that would be split: what the caller should bring.
extern "C" long llmrs_gemm_workspace_floats(int M, int N, int K) {
    if (M > 16 && M <= 64) {
        int s = few_rows_take_tiles(M, N, K) ? tiled_splits(M, N, K) : skinny_splits(N, K);
        return s > 1 ? (long)s * M * N : 0;
    }
    if (M >= 1024 && M % 256 > 16 && M % 256 <= 64 && K % 64 == 0 && (long)(M / 256) * ceil_div(N, 256) >= 160) {
        int s = skinny_splits(N, K);            // the rows beyond whole large tiles go to the kernel for few rows
        return s > 1 ? (long)s * (M % 256) * N : 0;
    }
    if (M > 64 && (long)ceil_div(M, 256) * ceil_div(N, 256) < 160) {
        int s = tiled_splits(M, N, K);
        long own = s > 1 ? (long)s * M * N : 0;
        // a few rows beyond whole 128-row tiles may go to the kernel for few rows, and the whole tiles be split then
        int over128 = M % 128;
        if (M >= 1024 && over128 > 0 && over128 <= 64 && K % 64 == 0)
            own = std::max(own, std::max(llmrs_gemm_workspace_floats(M - over128, N, K), llmrs_gemm_workspace_floats(over128, N, K)));
        return own;
    }
    return 0;
}

// Up to 16 rows a bfloat16 product goes to the kernel for few rows with every tile of a block finished by a wave
// of its own (not the widest weights, whose blocks take seven tiles): that kernel scales its rows' sums by a
// norm left to it and leaves what the next norm needs.
// Whether blocks of 24 features (a tile and a half) share a weight of N features out over the device's units more
// evenly, by a tenth of a round or more, than blocks of `whole` features (16 or 32) do.
static bool half_tile_blocks(int N, int whole, int cus) {
    auto even = [&](int b) { return (double)b / ((double)ceil_div(b, cus) * cus); };
    return N % 8 == 0 && even(ceil_div(N, 24)) > even(ceil_div(N, whole)) + 0.1;
}

extern "C" int llmrs_gemm_defers_norm(int M, int N, int K) { return M >= 1 && M <= 16 && N >= 1 && K % 8 == 0; }
// Up to 16 rows on a narrow weight with long rows (16-feature blocks would leave half of the compute units without
// one): blocks of 8 features, half a tile each (the tile's other rows are never asked for).  Measured at 1 row:
// 2048 x 8192 14.8 -> 12.3 us, 2048 x 2048 6.1 -> 5.6 us.
static bool half_blocks_for_narrow(int N, int K) {
    return N < 16384 && K >= 2048 && N % 8 == 0 && ceil_div(N, 16) * 2 <= llmrs_compute_units();
}
// How many partial sums of squares per row such a product leaves for the norm that follows (NextNorm without eps).
extern "C" int llmrs_gemm_next_parts(int M, int N, int K) {
    return M <= 16 && half_blocks_for_narrow(N, K) ? ceil_div(N, 8) : ceil_div(N, 16);
}
// 17 rows or more whose sums are split over blocks: the kernel that adds the parts up can finish the following norm.
// (Beyond 256 rows that is where the 128 x 128 tiles take all rows with k split: a narrow weight whose tiles leave
// half of the device's places empty, as the o and down products of a small model do beside a prompt portion.)
extern "C" int llmrs_gemm_norms_whole(int M, int N, int K) {
    if (!(M > 16 && N >= 4 && N % 4 == 0 && N <= 16384 && K % 8 == 0)) return 0;
    if (M <= 256) return llmrs_gemm_workspace_floats(M, N, K) > 0;
    return K % 64 == 0 && (long)ceil_div(M, 256) * ceil_div(N, 256) < 160 && tiled_splits(M, N, K) > 1;
}

// The product as parts of its sum over k, [parts][M][N] 32-bit in `workspace`, for a caller that adds them up itself
// (the rotation and cache write after the q/k/v product does, and saves the kernel that would): only where this
// file would split such a product over blocks anyway.  Returns the number of parts, 0 when the product is not
// one of those (nothing was launched), -1 on error.
int llmrs_gemm_bf16_split_parts(hipStream_t stream, const bf16* A, int lda, const bf16* W, int M, int N, int K,
                                void* workspace, size_t workspace_bytes) {
    if (K % 64 || lda % 8 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15) || workspace == nullptr || M > 512) return 0;
    const bool tiles = M > 64 ? !((long)ceil_div(M, 256) * ceil_div(N, 256) >= 160 && M > 128) : few_rows_take_tiles(M, N, K);
    int splits = tiles ? tiled_splits(M, N, K) : 1;
    if (splits <= 1 || workspace_bytes < (size_t)splits * M * N * sizeof(float)) return 0;
    if (launch_tiles_128(stream, A, lda, W, nullptr, N, M, N, K, LLMRS_EPI_STORE, splits, (float*)workspace, nullptr, false) != 0) return -1;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { llmrs_fail("gemm (mfma): launch failed: %s", hipGetErrorString(e)); return -1; }
    return splits;
}

int llmrs_gemm_bf16_mfma(hipStream_t stream, const bf16* A, int lda, const bf16* W, void* out, int ldc,
                         int M, int N, int K, int epi, void* workspace, size_t workspace_bytes,
                         const QkvEpilogue* qkv, const RowScale* scale, const NextNorm* next) {
    if (K % 8 || lda % 8 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) {
        if (scale != nullptr || next != nullptr) { llmrs_fail("gemm: a deferred norm needs rows of a multiple of 8 values, 16-byte aligned"); return -1; }
        return 0;
    }
    const bool whole = next != nullptr && next->eps > 0.0f;      // the norm that follows is finished by the kernel that adds the parts up
    if (whole) {
        bool ok = scale == nullptr && epi == LLMRS_EPI_ACCUM_F32 && llmrs_gemm_norms_whole(M, N, K) && workspace != nullptr &&
                  workspace_bytes >= (size_t)llmrs_gemm_workspace_floats(M, N, K) * sizeof(float) && next->y != nullptr &&
                  next->weight != nullptr && next->ldy >= N && next->ldy % 4 == 0 && ((uintptr_t)next->y & 7) == 0 &&
                  ((uintptr_t)next->weight & 15) == 0 && ldc % 4 == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)workspace & 15) == 0;
        if (!ok) { llmrs_fail("gemm: a norm finished by a split product needs the += epilogue, 17 rows or more of a shape that is split, its workspace and aligned rows, got M=%d N=%d K=%d epilogue %d", M, N, K, epi); return -1; }
    } else if (scale != nullptr || next != nullptr) {
        bool ok = llmrs_gemm_defers_norm(M, N, K) && (scale == nullptr || (scale->sumsq != nullptr && scale->nparts >= 1 && scale->eps > 0.0f)) &&
                  (next == nullptr || (epi == LLMRS_EPI_ACCUM_F32 && N < 16384 && next->sumsq != nullptr && next->y != nullptr &&
                                       next->weight != nullptr && next->ldy >= N && next->ldy % 4 == 0 && ((uintptr_t)next->y & 7) == 0));
        if (!ok) { llmrs_fail("gemm: a deferred norm is taken for up to 16 rows (what is left for the next one: with the += epilogue, under 16384 features), got M=%d N=%d K=%d epilogue %d", M, N, K, epi); return -1; }
    }
    if (epi == LLMRS_EPI_QKV) {   // only the skinny kernel fuses it; its 8-byte stores need aligned rows
        if (M > 64 || qkv == nullptr || qkv->head_dim % 4 || ldc % 4 || ((uintptr_t)out & 7) ||
            ((uintptr_t)qkv->k_cache & 7) || qkv->rotary_dim % 4)
            return 0;
        // long rows and many tokens: the tiles with k split over blocks are so much faster that
        // the separate rotation kernel is paid for (10240 x 8192 at 64 rows: 90 us fused, 51 + 6)
        // (with rows of 4096 the same route gains nothing: a decode step of the 8B shape at 64 requests 7.60 -> 7.55 ms,
        // at 40 and 48 requests none or a loss)
        if (M > 32 && K >= 8192 && few_rows_take_tiles(M, N, K)) return 0;
    }
    int rc = 0;
    bool tiles_for_few = false;
    if (epi != LLMRS_EPI_QKV && few_rows_take_tiles(M, N, K)) {
        int splits = tiled_splits(M, N, K);
        tiles_for_few = workspace != nullptr && workspace_bytes >= (size_t)splits * M * N * sizeof(float);
    }
    if (tiles_for_few) {
        rc = launch_tiles_128(stream, A, lda, W, out, ldc, M, N, K, epi, tiled_splits(M, N, K), (float*)workspace, next);
    } else if (M <= 64) {
        // Waves per block (NW) come from the weight's shape alone: k-blocks go to the
        // waves in turn and their sums are added in wave order, so for a given weight an
        // output's sum has one order whatever M, MT, NT and U are (up to 16 rows; with more, a
        // weight with few rows may have its k-blocks shared out over blocks as well).
        // Features per block (NT*16) grow with N and M: a block reads its tokens' rows
        // again for every 16*NT features, which costs L2 bandwidth once M is large, but
        // a weight with few rows needs small blocks to have enough of them.
        // (Measured on MI355X at the 8B shapes.)
        bool wide = N >= 16384;
        bool eight = !wide && K >= 2048;
        // A wide weight's blocks take 7 or 4 feature tiles: whichever number of blocks fills the
        // device's compute units more evenly (28672 features are 256 blocks of 7 tiles).  Its blocks
        // start their walk along k at staggered places, by groups of that many features.
        if (whole && skinny_splits(N, K) <= 1) { llmrs_fail("gemm: M=%d N=%d K=%d is not split after all: the norm cannot be finished here", M, N, K); return -1; }
        int cus = llmrs_compute_units();
        auto evenness = [&](int nt) { int b = ceil_div(N, 16 * nt); return (double)b / ((double)ceil_div(b, cus) * cus); };
        int wide_nt = (wide && evenness(7) >= evenness(4)) ? 7 : 4;
        // Other weights with long rows (measured at 8192 x 8192: 32.6 -> 28.6 us; nothing at K = 4096):
        // by groups of 64 features, which hold the features of any block that these weights get.
        int rot = wide ? 16 * wide_nt : (K >= 8192 ? 64 : 0);
#define SKINNY(MT, NT, NW, U) launch_skinny<MT, NT, NW, U>(stream, A, lda, W, out, ldc, M, N, K, epi, qkv, 1, nullptr, rot, scale, next)
        if (M <= 16) {
            if (wide) {
                // up to 4 rows blocks of 16 features (a decode step of eight 8B layers: 1.100 -> 1.086 ms at 3 rows,
                // 1.121 -> 1.116 at 4, slower from 6 on: every block reads the tokens' rows again)
                if (M <= 4) SKINNY(1, 1, 4, 8); else if (wide_nt == 7) SKINNY(1, 7, 4, 1); else SKINNY(1, 4, 4, 2);
            }
            else if (eight) {
                // Blocks of 16 features, unless they come to a round and a half of the device's units (6144 features on
                // 256: 384 blocks) and blocks of 24 to whole rounds: those, when nothing is to be left for a norm (which
                // counts its sums by 16 features)
                if (K >= 16384 && N >= 8192) SKINNY(1, 2, 8, 4);   // 8192 x 28672: 90 -> 83 us
                else if (half_blocks_for_narrow(N, K))
                    launch_skinny<1, 1, 8, 4, 8>(stream, A, lda, W, out, ldc, M, N, K, epi, qkv, 1, nullptr, rot, scale, next);
                else if (next == nullptr && half_tile_blocks(N, 16, cus))
                    launch_skinny<1, 2, 8, 4, 8>(stream, A, lda, W, out, ldc, M, N, K, epi, qkv, 1, nullptr, rot, scale, nullptr);
                else SKINNY(1, 1, 8, 4);
            }
            else SKINNY(1, 1, 4, 4);
        } else if (M <= 32) {
            int splits = skinny_splits(N, K);
            if (splits > 1 && epi != LLMRS_EPI_QKV && workspace != nullptr &&
                workspace_bytes >= (size_t)splits * M * N * sizeof(float)) {
                launch_skinny<2, 4, 8, 1>(stream, A, lda, W, out, ldc, M, N, K, epi, nullptr, splits, (float*)workspace, 0, nullptr, next);
            } else if (wide) { if (wide_nt == 7) SKINNY(2, 7, 4, 1); else SKINNY(2, 4, 4, 2); }
            else if (N > 4096) {
                if (eight && half_tile_blocks(N, 32, cus)) launch_skinny<2, 2, 8, 2, 8>(stream, A, lda, W, out, ldc, M, N, K, epi, qkv, 1, nullptr, rot);
                else if (eight) SKINNY(2, 2, 8, 2);
                else SKINNY(2, 2, 4, 2);
            }
            else { if (eight) SKINNY(2, 1, 8, 4); else SKINNY(2, 1, 4, 4); }
        } else {
            // 48 or 64 tokens and 64 features per block; when that leaves no more than 64 blocks, K is split
            // over blocks too, if the caller gave room for the partial sums (measured: it
            // pays for N = 4096, K = 14336, and no longer for N = 6144).
            auto rows_of = [&](auto tiles) {
                constexpr int MT = decltype(tiles)::value;
                int splits = skinny_splits(N, K);
                if (splits > 1 && epi != LLMRS_EPI_QKV && workspace != nullptr &&
                    workspace_bytes >= (size_t)splits * M * N * sizeof(float)) {
                    launch_skinny<MT, 4, 8, 1>(stream, A, lda, W, out, ldc, M, N, K, epi, nullptr, splits, (float*)workspace, 0, nullptr, next);
                } else if (wide) { if (wide_nt == 7) SKINNY(MT, 7, 4, 1); else SKINNY(MT, 4, 4, 2); }
                else if (N > 4096) {
                    if (eight && half_tile_blocks(N, 32, cus)) launch_skinny<MT, 2, 8, 1, 8>(stream, A, lda, W, out, ldc, M, N, K, epi, qkv, 1, nullptr, rot);
                    else if (eight) SKINNY(MT, 2, 8, 1);
                    else SKINNY(MT, 2, 4, 2);
                }
                else { if (eight) SKINNY(MT, 1, 8, 2); else SKINNY(MT, 1, 4, 2); }
            };
            if (M <= 48) rows_of(std::integral_constant<int, 3>{}); else rows_of(std::integral_constant<int, 4>{});
        }
#undef SKINNY
    } else {
        // K % 64 == 0: tiles loaded straight into LDS, two k-tiles of 64 there.  Other K: through
        // registers, with zero-filled tails.
        // 256 x 256 tiles of eight waves in two groups out of step (128 x 64 per wave: one LDS read
        // per MFMA less than the 64 x 64 per wave of the 128 x 128 tiles) where they fill most of the
        // device; else 128 x 128
        // tiles of four waves, two blocks to a compute unit, with the k range split over blocks when
        // even those are too few (measured on MI355X).
        // One large tile runs on a compute unit at a time, so a grid of them works in rounds and the
        // last round may be far from full (896 tiles on 256 units: 3.5 rounds cost 4).  Then the large
        // tiles get the features that make whole rounds and the small tiles, two to a unit, the rest.
        long m_tiles = ceil_div(M, 256), big_tiles = m_tiles * ceil_div(N, 256);
        int cus = llmrs_compute_units();
        // A few rows beyond whole tiles (a prompt portion of 2048 tokens beside 16 decoded ones)
        // would cost another row of tiles in full: they go to the kernel for few rows instead,
        // which reads the weight once more at memory speed.
        int over = M % 256;
        if (K % 64 == 0 && M >= 1024 && over > 0 && over <= 64 && (m_tiles - 1) * ceil_div(N, 256) >= 160) {
            size_t elt = (epi == LLMRS_EPI_STORE_F32 || epi == LLMRS_EPI_ACCUM_F32) ? sizeof(float) : sizeof(bf16);
            int whole_rows = M - over;
            rc = llmrs_gemm_bf16_mfma(stream, A, lda, W, out, ldc, whole_rows, N, K, epi, workspace, workspace_bytes, qkv);
            if (rc != 1) return rc;
            return llmrs_gemm_bf16_mfma(stream, A + (size_t)whole_rows * lda, lda, W, (char*)out + (size_t)whole_rows * ldc * elt,
                                        ldc, over, N, K, epi, workspace, workspace_bytes, qkv);
        }
        // (up to 128 rows a 256-row tile would be half empty; 257-384 rows are still faster on two rows of
        // large tiles than on three of small ones: the lm head at 300 rows 640 against 750 us)
        if (K % 64 == 0 && big_tiles >= 160 && M > 128) {
            // operands under 4 GB are read through buffer descriptors (32-bit offsets), 1-4 % faster
            const bool small = (size_t)M * lda * 2 < ((size_t)1 << 32) && (size_t)N * K * 2 < ((size_t)1 << 32);
            // square tiles: four waves with 128 x 128 outputs each where their epilogues and loads allow, else the
            // eight waves in two groups
            const bool four = small && fourwave_takes(epi, out, ldc, N);
            long whole = big_tiles / cus * cus, rest = big_tiles - whole;
            int n_split = (int)(whole / m_tiles) * 256;        // features of the whole rounds
            // (the features beyond whole rounds run on 128 x 128 tiles, two to a unit, a round of which takes about 0.62 of
            // a round of large tiles: when they come to more than one such round, a last round of large tiles that is
            // not full may be the shorter way: the o and down products at 6144 rows, 1.5 rounds of large tiles)
            long small_blocks = (long)ceil_div(N - n_split, 128) * ceil_div(M, 128);
            bool split_pays = (double)(whole / cus) + 0.62 * ceil_div(small_blocks, 2L * cus) < (double)ceil_div(big_tiles, (long)cus);
            if (n_split > 0 && n_split < N && rest > 0 && 2 * rest <= cus + cus / 4 && split_pays) {
                size_t elt = (epi == LLMRS_EPI_STORE_F32 || epi == LLMRS_EPI_ACCUM_F32) ? sizeof(float) : sizeof(bf16);
                void* out_rest = (char*)out + (size_t)(epi == LLMRS_EPI_SWIGLU ? n_split / 2 : n_split) * elt;
                rc = four && fourwave_takes(epi, out, ldc, n_split)
                         ? launch_fourwave<256, 256>(stream, A, lda, W, out, ldc, M, n_split, K, epi)
                     : small ? launch_pingpong<256, 256, 2, 4, true>(stream, A, lda, W, out, ldc, M, n_split, K, epi)
                             : launch_pingpong<256, 256, 2, 4, false>(stream, A, lda, W, out, ldc, M, n_split, K, epi);
                if (rc == 0) {
                    long wide_rest = m_tiles * ceil_div(N - n_split, 128);      // (256 x 128 tiles where they come to whole rounds, as below)
                    if (four && M >= 1024 && fourwave_takes(epi, out_rest, ldc, N - n_split) &&
                        10 * wide_rest >= 9 * (long)ceil_div(wide_rest, (long)cus) * cus)
                        rc = launch_fourwave<256, 128>(stream, A, lda, W + (size_t)n_split * K, out_rest, ldc, M, N - n_split, K, epi);
                    else
                        rc = launch_dma<128, 128, 2, 2, 2>(stream, A, lda, W + (size_t)n_split * K, out_rest, ldc, M, N - n_split, K, epi);
                }
            } else if (long t192 = m_tiles * ceil_div(N, 192); rest > 0 && t192 % cus == 0) {
                // 256 x 192 tiles where they come to whole rounds of the device and the square ones do not: the
                // q/k/v product of the 8B shape at 2048 rows is 192 square tiles on 256 units, or 256 of these
                // (eight waves of 64 x 96: in a prompt step 103 us, against 107 for four waves of 128 x 96)
                rc = small ? launch_pingpong<256, 192, 4, 2, true>(stream, A, lda, W, out, ldc, M, N, K, epi)
                           : launch_pingpong<256, 192, 4, 2, false>(stream, A, lda, W, out, ldc, M, N, K, epi);
            } else {
                rc = four ? launch_fourwave<256, 256>(stream, A, lda, W, out, ldc, M, N, K, epi)
                     : small ? launch_pingpong<256, 256, 2, 4, true>(stream, A, lda, W, out, ldc, M, N, K, epi)
                             : launch_pingpong<256, 256, 2, 4, false>(stream, A, lda, W, out, ldc, M, N, K, epi);
            }
        } else if (K % 64 == 0) {
            // The same for the 128 x 128 tiles, whose blocks run two to a compute unit: a few rows beyond whole
            // tiles that cost them another round of the device, or the split of k that filled it, go to the kernel
            // for few rows (the o and down products of the 8B shape: 2049 rows 526 -> about 350 us, 1025 rows 287 -> 240).
            // Counted in k-tiles that a place works through, round after round.
            int over128 = M % 128;
            if (M >= 1024 && over128 > 0 && over128 <= 64 && !whole && next == nullptr && scale == nullptr) {
                auto walk = [&](int rows) {
                    int s = tiled_splits(rows, N, K);
                    if (s > 1 && (workspace == nullptr || workspace_bytes < (size_t)s * rows * N * sizeof(float))) s = 1;
                    long blocks = (long)ceil_div(rows, 128) * ceil_div(N, 128) * s;
                    return ceil_div(blocks, (long)cus * 2) * (K / 64 / s);
                };
                if (walk(M) - walk(M - over128) >= 32) {
                    size_t elt = (epi == LLMRS_EPI_STORE_F32 || epi == LLMRS_EPI_ACCUM_F32) ? sizeof(float) : sizeof(bf16);
                    int whole_rows = M - over128;
                    rc = llmrs_gemm_bf16_mfma(stream, A, lda, W, out, ldc, whole_rows, N, K, epi, workspace, workspace_bytes, qkv);
                    if (rc != 1) return rc;
                    return llmrs_gemm_bf16_mfma(stream, A + (size_t)whole_rows * lda, lda, W, (char*)out + (size_t)whole_rows * ldc * elt,
                                                ldc, over128, N, K, epi, workspace, workspace_bytes, qkv);
                }
            }
            int splits = tiled_splits(M, N, K);
            // Many rows on a weight too narrow for the square tiles: four waves on 256 x 128 (128 x 64 a wave, a block
            // to a unit) where such tiles come to whole rounds of the device, or nearly: a k-step brings 48 KB into a
            // unit for the work that two 128 x 128 blocks bring 64 KB for (the o and down products of the 8B shape at
            // 2048 rows: a prompt step 31.55 -> 31.03 ms).
            long wide_blocks = (long)ceil_div(M, 256) * ceil_div(N, 128);
            const bool small4 = (size_t)M * lda * 2 < ((size_t)1 << 32) && (size_t)N * K * 2 < ((size_t)1 << 32);
            if (splits == 1 && !whole && next == nullptr && M >= 1024 && small4 && fourwave_takes(epi, out, ldc, N) &&
                10 * wide_blocks >= 9 * (long)ceil_div(wide_blocks, (long)cus) * cus)
                rc = launch_fourwave<256, 128>(stream, A, lda, W, out, ldc, M, N, K, epi);
            else if (splits > 1 && workspace != nullptr && workspace_bytes >= (size_t)splits * M * N * sizeof(float))
                rc = launch_tiles_128(stream, A, lda, W, out, ldc, M, N, K, epi, splits, (float*)workspace, next);
            else if (whole) rc = llmrs_fail("gemm: M=%d N=%d K=%d is not split after all: the norm cannot be finished here", M, N, K);
            else
                rc = launch_tiles_128(stream, A, lda, W, out, ldc, M, N, K, epi, 1, nullptr);
        }
        else rc = launch_tiled<128, 128, 64, 1>(stream, A, lda, W, out, ldc, M, N, K, epi);
    }
    if (rc != 0) return -1;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        llmrs_fail("gemm (mfma): launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 1;
}
