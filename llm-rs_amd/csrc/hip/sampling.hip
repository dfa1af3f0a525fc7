// Next-token choice on the device: only token ids go back to the host.
#include "common.h"

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
// Temperature / top-k / top-p sampling, one block per row.
//
// The reference does this on the host (src/sampler/mod.rs:84-154): logits * (1/T);
// all but the top_k largest dropped; softmax; the shortest prefix of the
// descending order whose mass reaches top_p kept and renormalised; then the
// first index, walking in index order, whose cumulative probability exceeds the
// request's uniform.  Here the same happens next to the logits:
//   * the k-th largest value by a radix select over order-preserving keys
//     (4 passes with a 256-bin histogram);
//   * with top_k <= MAX_CAND the survivors are gathered into LDS in index order
//     and one thread finishes the row exactly as the reference's loop does
//     (descending order, sequential 32-bit cumulative sums);
//   * without top_k (or a very large one) the top_p cut is found by a bitwise
//     search over keys with block-wide sums, and the draw by a scan over
//     contiguous segments.
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
// Sum of v over the threads before this one (thread order), and the total.
__device__ unsigned block_exclusive_scan_u(unsigned v, SampleShared& s, unsigned& total) {
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        unsigned o = __shfl_up(inc, off, 64);
        if (lane >= off) inc += o;
    }
    if (lane == 63) s.u[wave] = inc;
    __syncthreads();
    unsigned before = 0;
    total = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (w < wave) before += s.u[w];
        total += s.u[w];
    }
    __syncthreads();
    return before + inc - v;
}
__device__ float block_exclusive_scan_f(float v, SampleShared& s, float& total) {
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        float o = __shfl_up(inc, off, 64);
        if (lane >= off) inc += o;
    }
    if (lane == 63) s.f[wave] = inc;
    __syncthreads();
    float before = 0.0f;
    total = 0.0f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (w < wave) before += s.f[w];
        total += s.f[w];
    }
    __syncthreads();
    return before + (inc - v);
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

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits, int ld, int V,
                                                                     const int* __restrict__ words, int* __restrict__ out) {
    __shared__ SampleShared s;
    const float* row = logits + (size_t)blockIdx.x * ld;
    const int* w = words + 4 * blockIdx.x;
    float u = __int_as_float(w[0]), temp = __int_as_float(w[1]), top_p = __int_as_float(w[3]);
    int top_k = w[2];
    int tid = threadIdx.x;

    if (!(temp > 0.0f)) {   // greedy row: largest logit, lowest index on ties
        float best = -INFINITY;
        unsigned idx = 0xffffffffu;
        for (int i = tid; i < V; i += SAMPLE_THREADS) {
            float v = row[i];
            if (v > best || idx == 0xffffffffu) { best = v; idx = i; }
        }
        float m = block_max_f(best, s);
        unsigned first = block_min_u(best == m ? idx : 0xffffffffu, s);
        if (tid == 0) out[blockIdx.x] = first == 0xffffffffu ? 0 : (int)first;
        return;
    }

    float inv_t = 1.0f / temp;
    float zmax = -INFINITY;
    for (int i = tid; i < V; i += SAMPLE_THREADS) zmax = fmaxf(zmax, row[i] * inv_t);
    zmax = block_max_f(zmax, s);

    // ---- top_k: key of the k-th largest, and how many of its equals stay
    bool use_k = top_k > 0 && top_k < V;
    unsigned kth = 0, keep_eq_k = 0xffffffffu;   // keep: key > kth, or key == kth among the first keep_eq_k of them
    int cut_k = V;                               // ... that is, at indices <= cut_k
    if (use_k) {
        unsigned prefix = 0, mask = 0, remaining = top_k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int b = tid; b < 256; b += SAMPLE_THREADS) s.hist[b] = 0;
            __syncthreads();
            for (int i = tid; i < V; i += SAMPLE_THREADS) {
                unsigned k = order_key(row[i] * inv_t);
                if ((k & mask) == prefix) atomicAdd(&s.hist[(k >> shift) & 255], 1u);
            }
            __syncthreads();
            if (tid == 0) {
                unsigned seen = 0;
                int b = 255;
                for (; b > 0; --b) {
                    if (seen + s.hist[b] >= remaining) break;
                    seen += s.hist[b];
                }
                s.bcast[0] = (unsigned)b;
                s.bcast[1] = remaining - seen;   // still to take inside bin b
            }
            __syncthreads();
            prefix |= s.bcast[0] << shift;
            mask |= 255u << shift;
            remaining = s.bcast[1];
            __syncthreads();
        }
        kth = prefix;
        keep_eq_k = remaining;                   // >= 1
        unsigned n_eq = 0;
        for (int i = tid; i < V; i += SAMPLE_THREADS) n_eq += order_key(row[i] * inv_t) == kth;
        n_eq = block_sum_u(n_eq, s);
        if (n_eq > keep_eq_k) cut_k = index_cut(row, V, inv_t, kth, keep_eq_k, s);
    }
    auto kept_k = [&](unsigned k, int i) { return !use_k || k > kth || (k == kth && i <= cut_k); };

    int seg = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;     // contiguous indices per thread
    int lo = min(tid * seg, V), hi = min(lo + seg, V);

    if (use_k && top_k <= MAX_CAND) {
        // ---- survivors into LDS, in index order
        unsigned mine = 0;
        for (int i = lo; i < hi; ++i) mine += kept_k(order_key(row[i] * inv_t), i);
        unsigned total;
        unsigned at = block_exclusive_scan_u(mine, s, total);
        for (int i = lo; i < hi; ++i) {
            float z = row[i] * inv_t;
            if (kept_k(order_key(z), i)) { s.cand_z[at] = z; s.cand_i[at] = i; ++at; }
        }
        __syncthreads();
        if (tid == 0) {
            int n = (int)total;
            float sum = 0.0f;
            for (int c = 0; c < n; ++c) { s.cand_z[c] = expf(s.cand_z[c] - zmax); sum += s.cand_z[c]; }
            float inv = 1.0f / sum;
            for (int c = 0; c < n; ++c) s.cand_z[c] *= inv;           // probabilities
            if (top_p < 1.0f) {
                // walk in descending order (equal values: lower index first) until the mass reaches top_p
                float mass = 0.0f, last_p = INFINITY;
                int last_i = -1, taken = 0;
                while (taken < n) {
                    int best = -1;
                    for (int c = 0; c < n; ++c) {
                        float p = s.cand_z[c];
                        bool after_last = p < last_p || (p == last_p && s.cand_i[c] > last_i);
                        if (after_last && (best < 0 || p > s.cand_z[best])) best = c;
                    }
                    last_p = s.cand_z[best];
                    last_i = s.cand_i[best];
                    mass += last_p;
                    ++taken;
                    if (mass >= top_p) break;
                }
                float kept_sum = 0.0f;
                for (int c = 0; c < n; ++c) {
                    float p = s.cand_z[c];
                    bool keep = p > last_p || (p == last_p && s.cand_i[c] <= last_i);
                    if (!keep) s.cand_z[c] = 0.0f;
                    kept_sum += s.cand_z[c];
                }
                if (kept_sum > 0.0f) {
                    float inv2 = 1.0f / kept_sum;
                    for (int c = 0; c < n; ++c) s.cand_z[c] *= inv2;
                }
            }
            float cum = 0.0f;
            int pick = -1, last_kept = 0;
            for (int c = 0; c < n; ++c) {
                if (s.cand_z[c] > 0.0f) last_kept = s.cand_i[c];
                cum += s.cand_z[c];
                if (u < cum) { pick = s.cand_i[c]; break; }
            }
            out[blockIdx.x] = pick >= 0 ? pick : last_kept;
        }
        return;
    }

    // ---- no top_k (or a huge one): work on the whole row
    float mine = 0.0f;
    for (int i = lo; i < hi; ++i) {
        float z = row[i] * inv_t;
        if (kept_k(order_key(z), i)) mine += expf(z - zmax);
    }
    float S;
    block_exclusive_scan_f(mine, s, S);
    unsigned pth = 0;       // keep: key > pth, or key == pth at indices <= cut_p
    int cut_p = V;
    bool use_p = top_p < 1.0f;
    if (use_p) {
        float want = top_p * S;
        // largest key c with mass(key >= c) >= want, bit by bit
        unsigned prefix = 0;
        for (int bit = 31; bit >= 0; --bit) {
            unsigned cand = prefix | (1u << bit);
            float m = 0.0f;
            for (int i = lo; i < hi; ++i) {
                float z = row[i] * inv_t;
                unsigned k = order_key(z);
                if (k >= cand && kept_k(k, i)) m += expf(z - zmax);
            }
            float tot;
            block_exclusive_scan_f(m, s, tot);
            if (tot >= want) prefix = cand;
        }
        pth = prefix;
        float m_gt = 0.0f;
        unsigned n_eq = 0;
        for (int i = lo; i < hi; ++i) {
            float z = row[i] * inv_t;
            unsigned k = order_key(z);
            if (!kept_k(k, i)) continue;
            if (k > pth) m_gt += expf(z - zmax);
            n_eq += k == pth;
        }
        float mass_gt;
        block_exclusive_scan_f(m_gt, s, mass_gt);
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
    mine = 0.0f;
    int my_last = -1;
    for (int i = lo; i < hi; ++i) {
        float z = row[i] * inv_t;
        if (kept(order_key(z), i)) { mine += expf(z - zmax); my_last = i; }
    }
    float total;
    float before = block_exclusive_scan_f(mine, s, total);
    float target = u * total;
    unsigned owner = block_min_u((mine > 0.0f && target < before + mine) ? (unsigned)tid : 0xffffffffu, s);
    unsigned last_kept = 0;
    {   // the fallback when rounding leaves the uniform past the last sum
        unsigned v = my_last >= 0 ? (unsigned)(V - 1 - my_last) : 0xffffffffu;
        last_kept = V - 1 - block_min_u(v, s);
    }
    if (owner == 0xffffffffu) {
        if (tid == 0) out[blockIdx.x] = (int)last_kept;
        return;
    }
    if ((unsigned)tid == owner) {
        float cum = before;
        int pick = my_last;
        for (int i = lo; i < hi; ++i) {
            float z = row[i] * inv_t;
            if (!kept(order_key(z), i)) continue;
            cum += expf(z - zmax);
            if (target < cum) { pick = i; break; }
        }
        out[blockIdx.x] = pick;
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
