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
//   * top_k <= 1024 (the usual case): every thread takes the largest value of its
//     stretch of the row; the k-th largest of those 1024 maxima is a lower bound of
//     the k-th largest value of the row, so everything at or above it (a few
//     dozen values, typically) is gathered into LDS in index order, ranked there,
//     and cut to the k largest; one thread then finishes the row exactly as the
//     reference's loop does (descending order, sequential 32-bit cumulative sums).
//     Three passes over the row in all;
//   * a larger top_k: the k-th largest value by a radix select over order-preserving
//     keys (4 passes with a 256-bin histogram), survivors into LDS if they fit;
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
    unsigned char rank_drop[MAX_CAND];
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

// One thread finishes a row whose candidates lie in LDS in index order (those with
// rank_drop set are outside the top k): softmax, the top_p cut, the draw.
__device__ void finish_candidates(SampleShared& s, int n, float zmax, float top_p, float u, int* result) {
    float sum = 0.0f;
    for (int c = 0; c < n; ++c) {
        s.cand_z[c] = s.rank_drop[c] ? 0.0f : expf(s.cand_z[c] - zmax);
        sum += s.cand_z[c];
    }
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
    *result = pick >= 0 ? pick : last_kept;

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
    float mine_max = -INFINITY;
#pragma unroll 8
    for (int i = w_lo + lane; i < w_hi; i += 64) mine_max = fmaxf(mine_max, row[i] * inv_t);
    float zmax = block_max_f(mine_max, s);
    bool use_k = top_k > 0 && top_k < V;

    // Gathers the values with key >= bound (and index <= cut among those equal to `bound`, if
    // cut < V) into LDS in index order; returns how many there are (nothing is written if
    // they do not fit).
    auto gather = [&](unsigned bound, int cut) -> unsigned {
        auto in = [&](int i) { unsigned k = order_key(row[i] * inv_t); return k > bound || (k == bound && i <= cut); };
        unsigned cnt = 0;
    #pragma unroll 8
    for (int i = w_lo + lane; i < w_hi; i += 64) cnt += in(i);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, 64);
        unsigned total;
        unsigned base = wave_prefix_u(cnt, s, total);
        if (total > MAX_CAND) return total;
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

    if (use_k && top_k <= SAMPLE_THREADS) {
        // ---- a lower bound of the k-th largest value: the k-th largest of the threads' maxima
        unsigned mykey = w_lo + lane < w_hi ? order_key(mine_max) : 0u;
        unsigned prefix = 0, mask = 0, remaining = top_k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int b = tid; b < 256; b += SAMPLE_THREADS) s.hist[b] = 0;
            __syncthreads();
            if ((mykey & mask) == prefix) atomicAdd(&s.hist[(mykey >> shift) & 255], 1u);
            __syncthreads();
            if (tid == 0) {
                unsigned seen = 0;
                int b = 255;
                for (; b > 0; --b) {
                    if (seen + s.hist[b] >= remaining) break;
                    seen += s.hist[b];
                }
                s.bcast[0] = (unsigned)b;
                s.bcast[1] = remaining - seen;
            }
            __syncthreads();
            prefix |= s.bcast[0] << shift;
            mask |= 255u << shift;
            remaining = s.bcast[1];
            __syncthreads();
        }
        // at least top_k values of the row have a key >= prefix
        unsigned n = gather(prefix, V);
        if (n <= MAX_CAND) {
            // ---- the k largest of the candidates: a candidate's rank is the number of
            // candidates before it in the order (value descending, index ascending)
            for (int c = tid; c < (int)n; c += SAMPLE_THREADS) {
                float z = s.cand_z[c];
                int idx = s.cand_i[c], rank = 0;
                for (int j = 0; j < (int)n; ++j) {
                    float zj = s.cand_z[j];
                    rank += zj > z || (zj == z && s.cand_i[j] < idx);
                }
                s.rank_drop[c] = rank >= top_k;
            }
            __syncthreads();
            if (tid == 0) finish_candidates(s, (int)n, zmax, top_p, u, &out[blockIdx.x]);
            return;
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
        unsigned keep_eq = remaining;            // >= 1 of the values equal to the k-th stay
        unsigned n_eq = 0;
    #pragma unroll 8
    for (int i = w_lo + lane; i < w_hi; i += 64) n_eq += order_key(row[i] * inv_t) == kth;
        n_eq = block_sum_u(n_eq, s);
        if (n_eq > keep_eq) cut_k = index_cut(row, V, inv_t, kth, keep_eq, s);
        if (top_k <= MAX_CAND) {
            unsigned n = gather(kth, cut_k);     // exactly top_k values
            if (tid == 0) {
                for (int c = 0; c < (int)n; ++c) s.rank_drop[c] = 0;
                finish_candidates(s, (int)n, zmax, top_p, u, &out[blockIdx.x]);
            }
            return;
        }
    }
    auto kept_k = [&](unsigned k, int i) { return !use_k || k > kth || (k == kth && i <= cut_k); };

    // ---- no top_k (or a huge one): work on the whole row
    float mine = 0.0f;
#pragma unroll 8
    for (int i = w_lo + lane; i < w_hi; i += 64) {
        float z = row[i] * inv_t;
        if (kept_k(order_key(z), i)) mine += expf(z - zmax);
    }
    float S = block_sum_f(mine, s);
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
    if ((unsigned)wave != owner) return;
    float cum = before;
    int pick = -1, last_in_wave = -1;
    for (int i0 = w_lo; i0 < w_hi && pick < 0; i0 += 64) {
        int i = i0 + lane;
        float e = 0.0f;
        if (i < w_hi) {
            float z = row[i] * inv_t;
            if (kept(order_key(z), i)) e = expf(z - zmax);
        }
        float inc = e;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            float o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        unsigned long long hit = __ballot(e > 0.0f && target < cum + inc);
        unsigned long long any = __ballot(e > 0.0f);
        if (any) last_in_wave = i0 + 63 - __clzll(any);
        if (hit) pick = i0 + __ffsll((long long)hit) - 1;
        cum += __shfl(inc, 63, 64);
    }
    if (lane == 0) out[blockIdx.x] = pick >= 0 ? pick : last_in_wave;
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
