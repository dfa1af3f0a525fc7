// Next-token choice on the device: only token ids go back to the host.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

// Greedy: the index of the largest logit; of equal ones the lowest index wins.
// (The reference's kernel, shaders/ops.metal:803-835, leaves ties to the scan's
// shape and its host path takes the last maximum, src/sampler/mod.rs:65-68; a
// rule is chosen here so that kernel and plain implementation agree.)
__device__ __forceinline__ void argmax_merge(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

// Stage 1: block (row, part) scans its part of the row; stage 2 (part count 1, or
// the second launch over the partial results) picks among the parts.
#define ARGMAX_PARTS 32

__global__ __launch_bounds__(1024) void argmax_rows_kernel(const float* __restrict__ logits, int ld, int V,
                                                           const float* __restrict__ part_val,
                                                           const int* __restrict__ part_idx,
                                                           float* __restrict__ out_val, int* __restrict__ out_idx) {
    __shared__ float sv[16];
    __shared__ int si[16];
    int row = blockIdx.x, parts = gridDim.y, part = blockIdx.y;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    if (part_val == nullptr) {
        const float* src = logits + (size_t)row * ld;
        int per = (V + parts - 1) / parts;
        int lo = part * per, hi = min(lo + per, V);
        for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
            float v = src[i];
            if (v > best || idx == 0x7fffffff) { best = v; idx = i; }
        }
    } else {   // V is the number of partial results of this row
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            int pi = part_idx[row * V + i];
            if (pi != 0x7fffffff) argmax_merge(best, idx, part_val[row * V + i], pi);
        }
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
        if (out_val) { out_val[row * parts + part] = best; out_idx[row * parts + part] = idx; }
        else out_idx[row] = idx == 0x7fffffff ? 0 : idx;
    }
}

// scratch: room for n_rows * 32 (float, int) pairs, or null: then one block scans a whole row.
extern "C" int llmrs_argmax_rows(hipStream_t stream, const float* logits, int ld, int n_rows, int V, int* out,
                                 void* scratch, size_t scratch_bytes) {
    LLMRS_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax_rows: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    if (n_rows == 0) return 0;
    size_t need = (size_t)n_rows * ARGMAX_PARTS * 8;
    if (V >= 8192 && scratch != nullptr && scratch_bytes >= need) {
        float* pv = (float*)scratch;
        int* pi = (int*)(pv + (size_t)n_rows * ARGMAX_PARTS);
        argmax_rows_kernel<<<dim3(n_rows, ARGMAX_PARTS), 1024, 0, stream>>>(logits, ld, V, nullptr, nullptr, pv, pi);
        argmax_rows_kernel<<<dim3(n_rows, 1), 64, 0, stream>>>(nullptr, 0, ARGMAX_PARTS, pv, pi, nullptr, out);
    } else {
        argmax_rows_kernel<<<dim3(n_rows, 1), 1024, 0, stream>>>(logits, ld, V, nullptr, nullptr, nullptr, out);
    }
    LLMRS_LAUNCH_CHECK("argmax_rows");
    return 0;
}

// ---------------------------------------------------------------------------
// The same two stages for callers that cannot allocate (no_alloc.h): the partial
// results live in a file-scope array of device memory instead of a buffer the
// caller brings.  In host code the array's name only stands for the symbol; its
// address on a device is asked for once per device, with that device current,
// and kept.  Each GPU has its own copy of the array at its own address.
static __device__ __align__(256) unsigned char scratch[LLMRS_ARGMAX_STATIC_BYTES];
static_assert(LLMRS_ARGMAX_STATIC_BYTES == LLMRS_ARGMAX_STATIC_MAX_ROWS * ARGMAX_PARTS * 8, "a (value, index) pair per row and part");

#define LLMRS_MAX_DEVICES 64
static void* g_scratch_of_device[LLMRS_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int argmax_static_scratch(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    LLMRS_REQUIRE(e == hipSuccess, "argmax_rows_static: no current device: %s", hipGetErrorString(e));
    LLMRS_REQUIRE(dev >= 0 && dev < LLMRS_MAX_DEVICES, "argmax_rows_static: device %d is beyond the %d this library keeps addresses for",
                  dev, LLMRS_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_of_device[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        LLMRS_REQUIRE(e == hipSuccess && p != nullptr, "argmax_rows_static: cannot find the scratch array on device %d: %s", dev,
                      hipGetErrorString(e));
        g_scratch_of_device[dev] = p;
    }
    *ptr = g_scratch_of_device[dev];
    return 0;
}

// A call with n_rows = 0 only looks the array's address up: a caller that is about to
// record a graph makes one such call on each device first.
extern "C" int llmrs_argmax_rows_static(hipStream_t stream, const float* logits, int ld, int n_rows, int V, int* out) {
    LLMRS_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax_rows_static: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    LLMRS_REQUIRE(n_rows <= LLMRS_ARGMAX_STATIC_MAX_ROWS, "argmax_rows_static: %d rows, the scratch array holds the partial results of %d",
                  n_rows, LLMRS_ARGMAX_STATIC_MAX_ROWS);
    void* ptr = nullptr;
    if (argmax_static_scratch(&ptr) != 0) return -1;
    if (n_rows == 0) return 0;
    LLMRS_REQUIRE(logits != nullptr && out != nullptr, "argmax_rows_static: null logits or out");
    if (V >= 8192) {
        // Stage 1 writes every (row, part) pair that stage 2 reads, so what an earlier call left is never seen.
        float* pv = (float*)ptr;
        int* pi = (int*)(pv + (size_t)n_rows * ARGMAX_PARTS);
        argmax_rows_kernel<<<dim3(n_rows, ARGMAX_PARTS), 1024, 0, stream>>>(logits, ld, V, nullptr, nullptr, pv, pi);
        argmax_rows_kernel<<<dim3(n_rows, 1), 64, 0, stream>>>(nullptr, 0, ARGMAX_PARTS, pv, pi, nullptr, out);
    } else {
        argmax_rows_kernel<<<dim3(n_rows, 1), 1024, 0, stream>>>(logits, ld, V, nullptr, nullptr, nullptr, out);
    }
    LLMRS_LAUNCH_CHECK("argmax_rows_static");
    return 0;
}

// ---------------------------------------------------------------------------
// Temperature / top-k / top-p sampling, one block per row.
//
// The reference does this on the host (src/sampler/mod.rs:84-154): logits * (1/T);
// all but the top_k largest dropped; softmax; the shortest prefix of the
// descending order whose mass reaches top_p kept and renormalised; then the
// first index, walking in index order, whose cumulative probability exceeds the
// request's uniform.  Here the same happens next to the logits:
//   * top_k <= 1024 (the usual case): every thread takes the largest value of its
//     stretch of the row; the k-th largest of those 1024 maxima is a lower bound of
//     the k-th largest value of the row, so everything at or above it (a few
//     dozen values, typically) is gathered into LDS in index order, ranked there,
//     and cut to the k largest; the block then finishes the row as the reference's
//     loops do (descending order, sequential 32-bit cumulative sums by one thread; ranks,
//     exponentials and scalings shared out).  Three passes over the row in all;
//   * top_p without top_k: the same with the 512 largest values as candidates and the
//     softmax sum of the whole row taken in the gathering pass; if the top_p mass is
//     reached inside the candidates (any row but a flat one), the row is finished there;
//   * a larger top_k: the k-th largest value by a radix select over order-preserving
//     keys (4 passes with a 256-bin histogram), survivors into LDS if they fit;
//   * else (flat rows under top_p alone, a very large top_k) the top_p cut is found by a
//     bitwise search over keys with block-wide sums (32 passes: 0.7-0.9 ms on a row of
//     128 K), and the draw by a scan over contiguous segments, shared out twice.
// Of equal values at a cut the lowest indices stay (the reference's unstable
// sorts leave that open).  Every sum has a fixed order: a row's token depends on
// its logits and its uniform only.
// ---------------------------------------------------------------------------
#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / 64)
#define MAX_CAND 2048

__device__ __forceinline__ unsigned order_key(float z) {
    unsigned u = __float_as_uint(z);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(unsigned k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

struct SampleShared {
    float f[SAMPLE_WAVES];
    unsigned u[SAMPLE_WAVES];
    unsigned hist[256];
    unsigned bcast[4];
    float cand_z[MAX_CAND];
    int cand_i[MAX_CAND];
    float by_rank[MAX_CAND];
    unsigned short rank[MAX_CAND];
};

__device__ float block_sum_f(float v, SampleShared& s) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) s.f[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) t += s.f[w];
    __syncthreads();
    return t;
}
__device__ float block_max_f(float v, SampleShared& s) {
    v = wave_max(v);
    if ((threadIdx.x & 63) == 0) s.f[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = -INFINITY;
    for (int w = 0; w < SAMPLE_WAVES; ++w) t = fmaxf(t, s.f[w]);
    __syncthreads();
    return t;
}
__device__ unsigned block_sum_u(unsigned v, SampleShared& s) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) s.u[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned t = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) t += s.u[w];
    __syncthreads();
    return t;
}
__device__ unsigned block_min_u(unsigned v, SampleShared& s) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = min(v, (unsigned)__shfl_xor(v, off, 64));
    if ((threadIdx.x & 63) == 0) s.u[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned t = 0xffffffffu;
    for (int w = 0; w < SAMPLE_WAVES; ++w) t = min(t, s.u[w]);
    __syncthreads();
    return t;
}
// The histogram's bin in which the count, taken from bin 255 downwards, reaches `remaining`
// (bin 0 if it never does), and how many are still to take inside that bin: into bcast[0], bcast[1].
// The first wave does it, four bins a lane (a walk by one thread is a chain of 256 trips to LDS,
// 10 us a time).  The caller synchronises afterwards.
__device__ __forceinline__ void select_bin(SampleShared& s, unsigned remaining) {
    if (threadIdx.x >= 64) return;
    int lane = threadIdx.x;
    unsigned h[4], mine = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) { h[j] = s.hist[4 * lane + j]; mine += h[j]; }
    unsigned above = mine;                      // inclusive suffix sum over the lanes, then exclusive
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        unsigned o = __shfl_down(above, off, 64);
        if (lane + off < 64) above += o;
    }
    above -= mine;
    int bin = -1;
    unsigned left = 0, seen = above;
#pragma unroll
    for (int j = 3; j >= 0; --j) {
        if (bin < 0 && seen + h[j] >= remaining) { bin = 4 * lane + j; left = remaining - seen; }
        seen += h[j];
    }
    unsigned long long found = __ballot(bin >= 0);
    int top = found ? 63 - __clzll(found) : -1;  // the highest lane that holds a crossing: the first from above
    if (top < 0 || (top == 0 && __shfl(bin, 0, 64) == 0)) {
        // never reached above bin 0, or only inside it: bin 0, less everything above it
        if (lane == 0) { s.bcast[0] = 0u; s.bcast[1] = remaining - (above + mine - h[0]); }
    } else if (lane == top) {
        s.bcast[0] = (unsigned)bin;
        s.bcast[1] = left;
    }
}

// Smallest index c with exactly `need` elements of key `key` at indices <= c.
__device__ int index_cut(const float* row, int V, float inv_t, unsigned key, unsigned need, SampleShared& s) {
    int lo = 0, hi = V - 1;     // invariant: count(<= hi) >= need
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        unsigned c = 0;
        for (int i = threadIdx.x; i <= mid; i += SAMPLE_THREADS) c += order_key(row[i] * inv_t) == key;
        c = block_sum_u(c, s);
        if (c >= need) hi = mid; else lo = mid + 1;
    }
    return lo;
}

// The whole block finishes a row whose candidates lie in LDS in index order.  A candidate's rank
// is the number of candidates before it in the order (value descending, index ascending); those of
// rank >= top_k are outside.  Ranks, exponentials and scalings are shared out over the threads;
// every sum is one thread's, sequential and in 32 bits, as the reference's loops are: the softmax
// sum and the draw in index order, the top_p mass in descending order.
// `total` > 0: the softmax sum of the whole row, of which the candidates are the largest values
// (top_p without top_k); then, unless they are the whole row (`complete`), the top_p mass must be
// reached inside them: if it is not, nothing is written and false comes back (to every thread).
__device__ bool finish_candidates(SampleShared& s, int n, int top_k, float zmax, float top_p, float u, int* result,
                                  float total = 0.0f, bool complete = true) {
    int tid = threadIdx.x;
    for (int c = tid; c < n; c += SAMPLE_THREADS) {
        float z = s.cand_z[c];
        int idx = s.cand_i[c], rank = 0;
        for (int j = 0; j < n; ++j) {
            float zj = s.cand_z[j];
            rank += zj > z || (zj == z && s.cand_i[j] < idx);
        }
        s.rank[c] = (unsigned short)rank;
    }
    __syncthreads();
    for (int c = tid; c < n; c += SAMPLE_THREADS) s.cand_z[c] = s.rank[c] < top_k ? expf(s.cand_z[c] - zmax) : 0.0f;
    __syncthreads();
    if (tid == 0) {
        float sum = total;
        if (!(total > 0.0f)) {
            sum = 0.0f;
            for (int c = 0; c < n; ++c) sum += s.cand_z[c];
        }
        s.f[0] = 1.0f / sum;
    }
    __syncthreads();
    float inv = s.f[0];
    for (int c = tid; c < n; c += SAMPLE_THREADS) s.cand_z[c] *= inv;           // probabilities
    __syncthreads();
    if (top_p < 1.0f) {
        int m = min(n, top_k);                                                   // the candidates inside have ranks 0..m-1
        for (int c = tid; c < n; c += SAMPLE_THREADS)
            if (s.rank[c] < m) s.by_rank[s.rank[c]] = s.cand_z[c];
        __syncthreads();
        if (tid == 0) {     // descending order until the mass reaches top_p
            float mass = 0.0f;
            int last = 0;
            bool reached = false;
            for (; last < m; ++last) {
                mass += s.by_rank[last];
                if (mass >= top_p) { reached = true; break; }
            }
            s.bcast[0] = (unsigned)min(last, m - 1);
            s.bcast[1] = reached || complete;
        }
        __syncthreads();
        int last = (int)s.bcast[0];
        bool enough = s.bcast[1] != 0;
        __syncthreads();
        if (!enough) return false;
        for (int c = tid; c < n; c += SAMPLE_THREADS)
            if (s.rank[c] > last) s.cand_z[c] = 0.0f;
        __syncthreads();
        if (tid == 0) {
            float kept_sum = 0.0f;
            for (int c = 0; c < n; ++c) kept_sum += s.cand_z[c];
            s.f[0] = kept_sum > 0.0f ? 1.0f / kept_sum : 1.0f;
        }
        __syncthreads();
        float inv2 = s.f[0];
        for (int c = tid; c < n; c += SAMPLE_THREADS) s.cand_z[c] *= inv2;
        __syncthreads();
    }
    if (tid == 0) {
        float cum = 0.0f;
        int pick = -1, last_kept = 0;
        for (int c = 0; c < n; ++c) {
            if (s.cand_z[c] > 0.0f) last_kept = s.cand_i[c];
            cum += s.cand_z[c];
            if (u < cum) { pick = s.cand_i[c]; break; }
        }
        *result = pick >= 0 ? pick : last_kept;
    }
    return true;
}

// Exclusive prefix of v over the block's waves (wave order), and the total; v is a per-wave value.
__device__ unsigned wave_prefix_u(unsigned v, SampleShared& s, unsigned& total) {
    int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) s.u[wave] = v;
    __syncthreads();
    unsigned before = 0;
    total = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (w < wave) before += s.u[w];
        total += s.u[w];
    }
    __syncthreads();
    return before;
}
__device__ float wave_prefix_f(float v, SampleShared& s, float& total) {
    int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) s.f[wave] = v;
    __syncthreads();
    float before = 0.0f;
    total = 0.0f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (w < wave) before += s.f[w];
        total += s.f[w];
    }
    __syncthreads();
    return before;
}

// The row is shared out so that every read is coalesced and index order is (wave, round,
// lane): wave w owns the stretch [w_lo, w_hi) and reads it 64 consecutive values a round.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits, int ld, int V,
                                                                     const int* __restrict__ words, int* __restrict__ out) {
    __shared__ SampleShared s;
    const float* row = logits + (size_t)blockIdx.x * ld;
    const int* w = words + 4 * blockIdx.x;
    float u = __int_as_float(w[0]), temp = __int_as_float(w[1]), top_p = __int_as_float(w[3]);
    int top_k = w[2];
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int stretch = (((V + SAMPLE_WAVES - 1) / SAMPLE_WAVES) + 63) & ~63;
    int w_lo = min(wave * stretch, V), w_hi = min(w_lo + stretch, V);

    if (!(temp > 0.0f)) {   // greedy row: largest logit, lowest index on ties
        float best = -INFINITY;
        unsigned idx = 0xffffffffu;
#pragma unroll 8
        for (int i = w_lo + lane; i < w_hi; i += 64) {
            float v = row[i];
            if (v > best || idx == 0xffffffffu) { best = v; idx = i; }
        }
        float m = block_max_f(best, s);
        unsigned first = block_min_u(best == m ? idx : 0xffffffffu, s);
        if (tid == 0) out[blockIdx.x] = first == 0xffffffffu ? 0 : (int)first;
        return;
    }

    float inv_t = 1.0f / temp;
    // Rows that allow it are read 16 bytes a lane (a wave's round is 256 consecutive values, a lane's
    // four of them consecutive): four times the bytes in flight of a block that has a row to itself.
    bool vec = (((uintptr_t)row | (uintptr_t)V) & 3) == 0 && ((uintptr_t)row & 15) == 0;
    float mine_max = -INFINITY;        // largest value of this thread's share (any sharing out will do here)
    bool mine_any = false;
    if (vec) {
        const float4* row4 = (const float4*)row;
#pragma unroll 4
        for (int i = tid; i < (V >> 2); i += SAMPLE_THREADS) {
            float4 v = row4[i];
            mine_max = fmaxf(fmaxf(mine_max, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
            mine_any = true;
        }
    } else {
#pragma unroll 8
        for (int i = w_lo + lane; i < w_hi; i += 64) { mine_max = fmaxf(mine_max, row[i]); mine_any = true; }
    }
    mine_max *= inv_t;                 // scaling keeps the order: the largest scaled value is the scaled largest
    float zmax = block_max_f(mine_max, s);
    bool use_k = top_k > 0 && top_k < V;

    // Gathers the values with key >= bound (and index <= cut among those equal to `bound`, if
    // cut < V) into LDS in index order; returns how many there are (nothing is written if
    // they do not fit).
    auto gather = [&](unsigned bound, int cut, float* row_mass = nullptr) -> unsigned {
        auto in = [&](int i) { unsigned k = order_key(row[i] * inv_t); return k > bound || (k == bound && i <= cut); };
        auto in_z = [&](float z, int i) { unsigned k = order_key(z); return k > bound || (k == bound && i <= cut); };
        unsigned cnt = 0;
        float mass = 0.0f;      // with row_mass: the softmax sum of the whole row, in the same pass
        if (vec) {      // (w_lo and w_hi are multiples of 4 here: V is, and the stretches are multiples of 64)
#pragma unroll 4
            for (int i = w_lo + lane * 4; i < w_hi; i += 256) {
                float4 v = *(const float4*)(row + i);
                float z0 = v.x * inv_t, z1 = v.y * inv_t, z2 = v.z * inv_t, z3 = v.w * inv_t;
                cnt += in_z(z0, i) + in_z(z1, i + 1) + in_z(z2, i + 2) + in_z(z3, i + 3);
                if (row_mass) mass += (expf(z0 - zmax) + expf(z1 - zmax)) + (expf(z2 - zmax) + expf(z3 - zmax));
            }
        } else {
#pragma unroll 8
            for (int i = w_lo + lane; i < w_hi; i += 64) {
                cnt += in(i);
                if (row_mass) mass += expf(row[i] * inv_t - zmax);
            }
        }
        if (row_mass) *row_mass = block_sum_f(mass, s);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, 64);
        unsigned total;
        unsigned base = wave_prefix_u(cnt, s, total);
        if (total > MAX_CAND) return total;
        if (vec) {
            unsigned long long below = (1ull << lane) - 1ull;
            for (int i0 = w_lo; i0 < w_hi; i0 += 256) {
                int i = i0 + lane * 4;
                bool ok = i < w_hi;
                float4 v = ok ? *(const float4*)(row + i) : float4{0.f, 0.f, 0.f, 0.f};
                float z[4] = {v.x * inv_t, v.y * inv_t, v.z * inv_t, v.w * inv_t};
                bool f[4];
                unsigned long long b[4];
                unsigned at = base;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    f[j] = ok && in_z(z[j], i + j);
                    b[j] = __ballot(f[j]);
                    at += __popcll(b[j] & below);          // those of the lanes before this one
                    base += __popcll(b[j]);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (f[j]) { s.cand_z[at] = z[j]; s.cand_i[at] = i + j; ++at; }
            }
            __syncthreads();
            return total;
        }
        for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
            int i = i0 + lane;
            bool p = i < w_hi && in(i);
            unsigned long long b = __ballot(p);
            if (p) {
                unsigned at = base + __popcll(b & ((1ull << lane) - 1ull));
                s.cand_z[at] = row[i] * inv_t;
                s.cand_i[at] = i;
            }
            base += __popcll(b);
        }
        __syncthreads();
        return total;
    };

    // top_p alone: the values that matter are the largest few hundred in all rows but flat ones.  The 512
    // largest (and what else is no smaller than the bound below) become candidates; if the top_p mass
    // is reached inside them, the row is finished there; if not, by the search over the whole row below.
    bool nucleus_try = !use_k && top_p < 1.0f;
    if ((use_k && top_k <= SAMPLE_THREADS) || nucleus_try) {
        // ---- a lower bound of the k-th largest value: the k-th largest of the threads' maxima
        unsigned mykey = mine_any ? order_key(mine_max) : 0u;
        unsigned prefix = 0, mask = 0, remaining = use_k ? top_k : 512;
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int b = tid; b < 256; b += SAMPLE_THREADS) s.hist[b] = 0;
            __syncthreads();
            if ((mykey & mask) == prefix) atomicAdd(&s.hist[(mykey >> shift) & 255], 1u);
            __syncthreads();
            select_bin(s, remaining);
            __syncthreads();
            prefix |= s.bcast[0] << shift;
            mask |= 255u << shift;
            remaining = s.bcast[1];
            __syncthreads();
        }
        // at least top_k values of the row have a key >= prefix
        float row_mass = 0.0f;
        unsigned n = gather(prefix, V, nucleus_try ? &row_mass : nullptr);
        if (n <= MAX_CAND) {    // the k largest of the candidates, and the rest of the row's work, in LDS
            if (!nucleus_try) {
                finish_candidates(s, (int)n, top_k, zmax, top_p, u, &out[blockIdx.x]);
                return;
            }
            if (finish_candidates(s, (int)n, (int)n, zmax, top_p, u, &out[blockIdx.x], row_mass, (int)n == V)) return;
        }
        // too many equal or near values: the general path below handles it
    }

    // ---- top_k in general: key of the k-th largest by radix select, and how many of its equals stay
    unsigned kth = 0;
    int cut_k = V;             // keep: key > kth, or key == kth at indices <= cut_k
    if (use_k) {
        unsigned prefix = 0, mask = 0, remaining = top_k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int b = tid; b < 256; b += SAMPLE_THREADS) s.hist[b] = 0;
            __syncthreads();
#pragma unroll 8
            for (int i = w_lo + lane; i < w_hi; i += 64) {
                unsigned k = order_key(row[i] * inv_t);
                if ((k & mask) == prefix) atomicAdd(&s.hist[(k >> shift) & 255], 1u);
            }
            __syncthreads();
            select_bin(s, remaining);
            __syncthreads();
            prefix |= s.bcast[0] << shift;
            mask |= 255u << shift;
            remaining = s.bcast[1];
            __syncthreads();
        }
        kth = prefix;
        unsigned keep_eq = remaining;            // >= 1 of the values equal to the k-th stay
        unsigned n_eq = 0;
#pragma unroll 8
        for (int i = w_lo + lane; i < w_hi; i += 64) n_eq += order_key(row[i] * inv_t) == kth;
        n_eq = block_sum_u(n_eq, s);
        if (n_eq > keep_eq) cut_k = index_cut(row, V, inv_t, kth, keep_eq, s);
        if (top_k <= MAX_CAND) {
            unsigned n = gather(kth, cut_k);     // exactly top_k values
            finish_candidates(s, (int)n, (int)n, zmax, top_p, u, &out[blockIdx.x]);
            return;
        }
    }
    auto kept_k = [&](unsigned k, int i) { return !use_k || k > kth || (k == kth && i <= cut_k); };

    // ---- no top_k (or a huge one): work on the whole row
    float mine = 0.0f;
    unsigned pth = 0;       // keep: key > pth, or key == pth at indices <= cut_p
    int cut_p = V;
    bool use_p = top_p < 1.0f;
    if (use_p) {
#pragma unroll 8
        for (int i = w_lo + lane; i < w_hi; i += 64) {
            float z = row[i] * inv_t;
            if (kept_k(order_key(z), i)) mine += expf(z - zmax);
        }
        float S = block_sum_f(mine, s);
        float want = top_p * S;
        // largest key c with mass(key >= c) >= want, bit by bit
        unsigned prefix = 0;
        for (int bit = 31; bit >= 0; --bit) {
            unsigned cand = prefix | (1u << bit);
            float m = 0.0f;
#pragma unroll 8
            for (int i = w_lo + lane; i < w_hi; i += 64) {
                float z = row[i] * inv_t;
                unsigned k = order_key(z);
                if (k >= cand && kept_k(k, i)) m += expf(z - zmax);
            }
            if (block_sum_f(m, s) >= want) prefix = cand;
        }
        pth = prefix;
        float m_gt = 0.0f;
        unsigned n_eq = 0;
#pragma unroll 8
        for (int i = w_lo + lane; i < w_hi; i += 64) {
            float z = row[i] * inv_t;
            unsigned k = order_key(z);
            if (!kept_k(k, i)) continue;
            if (k > pth) m_gt += expf(z - zmax);
            n_eq += k == pth;
        }
        float mass_gt = block_sum_f(m_gt, s);
        n_eq = block_sum_u(n_eq, s);
        float e = expf(key_value(pth) - zmax);
        unsigned need = 1;
        float mass = mass_gt + e;
        while (mass < want && need < n_eq) { mass += e; ++need; }
        if (need < n_eq) cut_p = index_cut(row, V, inv_t, pth, need, s);
    }
    auto kept = [&](unsigned k, int i) {
        if (!kept_k(k, i)) return false;
        return !use_p || k > pth || (k == pth && i <= cut_p);
    };
    // ---- the draw: which wave's stretch holds the uniform, then a walk through that stretch
    mine = 0.0f;
    int my_last = -1;
#pragma unroll 8
    for (int i = w_lo + lane; i < w_hi; i += 64) {
        float z = row[i] * inv_t;
        if (kept(order_key(z), i)) { mine += expf(z - zmax); my_last = max(my_last, i); }
    }
    float wave_mass = wave_sum(mine);
    float total;
    float before = wave_prefix_f(wave_mass, s, total);
    float target = u * total;
    unsigned last_kept = V - 1 - block_min_u(my_last >= 0 ? (unsigned)(V - 1 - my_last) : 0xffffffffu, s);
    unsigned owner = block_min_u((wave_mass > 0.0f && target < before + wave_mass) ? (unsigned)wave : 0xffffffffu, s);
    if (owner == 0xffffffffu) {   // rounding left the uniform past the last sum
        if (tid == 0) out[blockIdx.x] = (int)last_kept;
        return;
    }
    // ---- the owner's stretch is shared out over all waves once more (a walk through all of it by one
    // wave is a hundred rounds, one after the other): sub-stretches of at most WALK rounds, their
    // masses, the one that holds the uniform, and a walk through that one from registers.
    constexpr int WALK = 8;
    if ((unsigned)wave == owner && lane == 0) s.bcast[0] = __float_as_uint(before);
    __syncthreads();
    float cum = __uint_as_float(s.bcast[0]);
    __syncthreads();
    int o_lo = min((int)owner * stretch, V), o_hi = min(o_lo + stretch, V);
    int pick = -1;
    while (pick < 0) {      // (one turn unless the stretch is longer than 16 * WALK rounds: then sub-stretch by sub-stretch)
        int span = min(o_hi - o_lo, SAMPLE_WAVES * WALK * 64);
        int sub = (((span + SAMPLE_WAVES - 1) / SAMPLE_WAVES) + 63) & ~63;
        int s_lo = min(o_lo + wave * sub, o_lo + span), s_hi = min(s_lo + sub, o_lo + span);
        float es[WALK];
        float part = 0.0f;
        int my_sub_last = -1;
#pragma unroll
        for (int r = 0; r < WALK; ++r) {
            int i = s_lo + 64 * r + lane;
            es[r] = 0.0f;
            if (i < s_hi) {
                float z = row[i] * inv_t;
                if (kept(order_key(z), i)) { es[r] = expf(z - zmax); my_sub_last = i; }
            }
            part += es[r];
        }
        float sub_mass = wave_sum(part);
        float sub_total;
        float sub_before = wave_prefix_f(sub_mass, s, sub_total);
        unsigned sub_owner = block_min_u((sub_mass > 0.0f && target < cum + sub_before + sub_mass) ? (unsigned)wave : 0xffffffffu, s);
        unsigned sub_last = V - 1 - block_min_u(my_sub_last >= 0 ? (unsigned)(V - 1 - my_sub_last) : 0xffffffffu, s);
        if (sub_owner == 0xffffffffu) {
            if (o_lo + span >= o_hi) {          // rounding left the uniform past the stretch's last sum
                if (tid == 0) out[blockIdx.x] = sub_last < (unsigned)V ? (int)sub_last : (int)last_kept;
                return;
            }
            cum += sub_total;                   // not in this part of the stretch: on to the next
            o_lo += span;
            continue;
        }
        if ((unsigned)wave != sub_owner) return;
        float c = cum + sub_before;
        int last_in_wave = -1;
#pragma unroll
        for (int r = 0; r < WALK; ++r) {
            int i0 = s_lo + 64 * r;
            if (pick >= 0) break;
            float e = es[r], inc = e;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                float o = __shfl_up(inc, off, 64);
                if (lane >= off) inc += o;
            }
            unsigned long long hit = __ballot(e > 0.0f && target < c + inc);
            unsigned long long any = __ballot(e > 0.0f);
            if (any) last_in_wave = i0 + 63 - __clzll(any);
            if (hit) pick = i0 + __ffsll((long long)hit) - 1;
            c += __shfl(inc, 63, 64);
        }
        if (pick < 0) pick = last_in_wave;      // rounding again: the sub-stretch's last kept value
        if (lane == 0) out[blockIdx.x] = pick;
        return;
    }
}

// words: [n_rows, 4] = uniform (float bits), temperature (float bits), top_k, top_p (float bits)
extern "C" int llmrs_sample_rows(hipStream_t stream, const float* logits, int ld, int n_rows, int V,
                                 const int* words, int* out) {
    LLMRS_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "sample_rows: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    if (n_rows == 0) return 0;
    sample_rows_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, words, out);
    LLMRS_LAUNCH_CHECK("sample_rows");
    return 0;
}

// tokens[rows[i]] = ids[sources[i]] for i < n: the ids a step sampled go into the next step's token array on the
// device, for a caller that starts that step before the ids have reached the host.  rows are places in `tokens`
// (n_tokens long), sources rows of `ids` (n_ids long); a pair outside either is left alone, and so is an id outside
// the vocabulary (the token then stays what the host wrote there).
__global__ void place_ids_kernel(int* __restrict__ tokens, int n_tokens, const int* __restrict__ rows,
                                 const int* __restrict__ sources, const int* __restrict__ ids, int n_ids, int n, int V) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int row = rows[i], src = sources[i];
    if (row < 0 || row >= n_tokens || src < 0 || src >= n_ids) return;
    int id = ids[src];
    if (id >= 0 && id < V) tokens[row] = id;
}

extern "C" int llmrs_place_ids(hipStream_t stream, int* tokens, int n_tokens, const int* rows, const int* sources,
                               const int* ids, int n_ids, int n, int V) {
    LLMRS_REQUIRE(n >= 0 && n_tokens >= 0 && n_ids >= 0 && V > 0, "place_ids: bad sizes n=%d tokens=%d ids=%d V=%d", n, n_tokens, n_ids, V);
    if (n == 0) return 0;
    LLMRS_REQUIRE(tokens && rows && sources && ids, "place_ids: null argument");
    place_ids_kernel<<<(n + 255) / 256, 256, 0, stream>>>(tokens, n_tokens, rows, sources, ids, n_ids, n, V);
    LLMRS_LAUNCH_CHECK("place_ids");
    return 0;
}
