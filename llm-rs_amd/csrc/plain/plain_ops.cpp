// Plain C++ twins of the device kernels: for every entry point of the kernel library a function with the same
// arguments (the stream first, ignored; pointers are host memory), written as the loops of the formulas,
// one output at a time, sums in double precision, one rounding on the way out.  They are the second oracle
// of the kernel tests (the first is the float64 PyTorch implementation under tests/): nothing in the package
// loads this library, there is no CPU path.
//
// Formulas: shaders/ops.metal:970-1003 (RMSNorm), :1011-1042 (rotation), :841-853 (cache write), :636-758
// (attention over pages), :803-835 (argmax); src/sampler/mod.rs:84-154 (sampling); src/arch/llama.rs:128-171
// (what the products feed).
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <vector>

namespace {

enum { F32 = 0, BF16 = 1 };
enum { EPI_STORE = 0, EPI_STORE_F32 = 1, EPI_ACCUM_F32 = 2, EPI_SWIGLU = 3 };

inline float bf16_to_float(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
// round to nearest, ties to even
inline uint16_t float_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);   // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
inline double load(const void* p, int dtype, size_t i) {
    return dtype == BF16 ? (double)bf16_to_float(((const uint16_t*)p)[i]) : (double)((const float*)p)[i];
}
inline void store(void* p, int dtype, size_t i, double v) {
    if (dtype == BF16) ((uint16_t*)p)[i] = float_to_bf16((float)v);
    else ((float*)p)[i] = (float)v;
}
inline bool known(int dtype) { return dtype == F32 || dtype == BF16; }
inline float bits_to_float(int w) {
    float f;
    std::memcpy(&f, &w, 4);
    return f;
}

// keys [page][kv_head][slot][feature], values [page][kv_head][feature][slot]
inline size_t key_at(int page, int kvh, int slot, int d, int n_kv, int ps, int hd) {
    return (((size_t)page * n_kv + kvh) * ps + slot) * hd + d;
}
inline size_t value_at(int page, int kvh, int slot, int d, int n_kv, int ps, int hd) {
    return (((size_t)page * n_kv + kvh) * hd + d) * ps + slot;
}

// The two features of rotation pair i of a head, and whether the pair is rotated at all.
inline void pair_of(int i, int rotary_dim, int interleaved, int& da, int& db, bool& rotated) {
    rotated = i < rotary_dim / 2;
    if (rotated) {
        if (interleaved) { da = 2 * i; db = 2 * i + 1; }
        else { da = i; db = i + rotary_dim / 2; }
    } else {
        da = rotary_dim + 2 * (i - rotary_dim / 2);
        db = da + 1;
    }
}

}  // namespace

// out[t, :] = table[tokens[t], :] * scale, 32-bit
extern "C" int llmrs_plain_embed_rows(void*, int dtype, float* out, const void* table, const int* tokens, int n_tokens,
                                      int D, int V, float scale) {
    if (!known(dtype) || n_tokens < 0 || D <= 0 || V <= 0) return -1;
    for (int t = 0; t < n_tokens; ++t) {
        if (tokens[t] < 0 || tokens[t] >= V) return -1;
        for (int d = 0; d < D; ++d) out[(size_t)t * D + d] = (float)(load(table, dtype, (size_t)tokens[t] * D + d) * (double)scale);
    }
    return 0;
}

// out[i, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * weight, r = rows[i] (rows null: r = i)
extern "C" int llmrs_plain_rmsnorm(void*, int dtype, void* out, const float* x, const float* weight, const int* rows,
                                   int n_rows, int D, float eps) {
    if (!known(dtype) || n_rows < 0 || D <= 0) return -1;
    for (int i = 0; i < n_rows; ++i) {
        const float* row = x + (size_t)(rows ? rows[i] : i) * D;
        double ss = 0.0;
        for (int d = 0; d < D; ++d) ss += (double)row[d] * row[d];
        double inv = 1.0 / std::sqrt(ss / D + (double)eps);
        for (int d = 0; d < D; ++d) store(out, dtype, (size_t)i * D + d, row[d] * inv * weight[d]);
    }
    return 0;
}

// C[m, n] = sum_k A[m, k] W[n, k], then the epilogue.  scale_sumsq: each row's sum is multiplied by
// 1 / sqrt(sum_p scale_sumsq[m, p] / K + scale_eps) (a norm left to this product).  next_y (with the += epilogue):
// what the following norm needs of the stream's new rows: with next_eps > 0 the normed rows themselves,
// else the rows times the norm's weight and, in next_sumsq, the sums of squares of each 16 features.
extern "C" int llmrs_plain_gemm(void*, int dtype, const void* A, int lda, const void* W, void* out, int ldc, int M, int N,
                                int K, int epi, void*, size_t, int, const float* scale_sumsq, int scale_parts,
                                float scale_eps, float* next_sumsq, void* next_y, int next_ldy, const float* next_weight,
                                float next_eps) {
    if (!known(dtype) || M < 0 || N <= 0 || K <= 0 || lda < K || epi < 0 || epi > 3) return -1;
    if (epi == EPI_SWIGLU && (N % 2 || ldc < N / 2)) return -1;
    if (epi != EPI_SWIGLU && ldc < N) return -1;
    if (next_y != nullptr && epi != EPI_ACCUM_F32) return -1;
    std::vector<double> sums(N);
    for (int m = 0; m < M; ++m) {
        double inv = 1.0;
        if (scale_sumsq != nullptr) {
            double ss = 0.0;
            for (int p = 0; p < scale_parts; ++p) ss += scale_sumsq[(size_t)m * scale_parts + p];
            inv = 1.0 / std::sqrt(ss / K + (double)scale_eps);
        }
        for (int n = 0; n < N; ++n) {
            double s = 0.0;
            for (int k = 0; k < K; ++k) s += load(A, dtype, (size_t)m * lda + k) * load(W, dtype, (size_t)n * K + k);
            sums[n] = s * inv;
        }
        if (epi == EPI_STORE) {
            for (int n = 0; n < N; ++n) store(out, dtype, (size_t)m * ldc + n, sums[n]);
        } else if (epi == EPI_STORE_F32) {
            for (int n = 0; n < N; ++n) ((float*)out)[(size_t)m * ldc + n] = (float)sums[n];
        } else if (epi == EPI_ACCUM_F32) {
            float* o = (float*)out + (size_t)m * ldc;
            for (int n = 0; n < N; ++n) o[n] = (float)((double)o[n] + sums[n]);
            if (next_y != nullptr) {
                double ss = 0.0;
                for (int n = 0; n < N; ++n) ss += (double)o[n] * o[n];
                double rinv = next_eps > 0.0f ? 1.0 / std::sqrt(ss / N + (double)next_eps) : 1.0;
                for (int n = 0; n < N; ++n)
                    ((uint16_t*)next_y)[(size_t)m * next_ldy + n] = float_to_bf16((float)((double)o[n] * rinv * next_weight[n]));
                if (!(next_eps > 0.0f) && next_sumsq != nullptr) {
                    int parts = (N + 15) / 16;
                    for (int p = 0; p < parts; ++p) {
                        double part = 0.0;
                        for (int n = 16 * p; n < std::min(N, 16 * p + 16); ++n) part += (double)o[n] * o[n];
                        next_sumsq[(size_t)m * parts + p] = (float)part;
                    }
                }
            }
        } else {   // rows of W are (gate_0, up_0, gate_1, up_1, ...): silu(gate) * up
            for (int n = 0; n < N; n += 2) {
                double g = sums[n], u = sums[n + 1];
                store(out, dtype, (size_t)m * ldc + n / 2, g / (1.0 + std::exp(-g)) * u);
            }
        }
    }
    return 0;
}

// Rotates q (in place) and k by angle = position * inv_freq[i] for pair i of each head, and writes k (rotated) and
// v into the cache at slot_map[t] = page * page_size + slot.  k and v stay as they are in qkv.
extern "C" int llmrs_plain_rope_kv_write(void*, int dtype, void* qkv, int row_stride, const int* positions,
                                         const int* slot_map, const float* inv_freq, int rotary_dim, int interleaved,
                                         void* k_cache, void* v_cache, int n_tokens, int n_heads, int n_kv_heads,
                                         int head_dim, int page_size, int num_pages, int write_kv) {
    if (!known(dtype) || head_dim % 2 || rotary_dim % 2 || rotary_dim > head_dim || rotary_dim < 0) return -1;
    int heads = n_heads + 2 * n_kv_heads;
    for (int t = 0; t < n_tokens; ++t)
        for (int head = 0; head < heads; ++head) {
            bool is_q = head < n_heads, is_k = !is_q && head < n_heads + n_kv_heads;
            if (!is_q && !write_kv) continue;
            size_t base = (size_t)t * row_stride + (size_t)head * head_dim;
            int slot = is_q ? 0 : slot_map[t];
            if (!is_q && (slot < 0 || slot >= num_pages * page_size)) continue;
            for (int i = 0; i < head_dim / 2; ++i) {
                int da, db;
                bool rotated;
                pair_of(i, rotary_dim, interleaved, da, db, rotated);
                double a = load(qkv, dtype, base + da), b = load(qkv, dtype, base + db);
                if (rotated && (is_q || is_k)) {
                    double angle = (double)((float)positions[t] * inv_freq[i]);     // the angle itself is a 32-bit product
                    double c = std::cos(angle), s = std::sin(angle);
                    double ya = a * c - b * s, yb = a * s + b * c;
                    a = ya; b = yb;
                }
                if (is_q) {
                    store(qkv, dtype, base + da, a);
                    store(qkv, dtype, base + db, b);
                } else if (is_k) {
                    int kvh = head - n_heads;
                    store(k_cache, dtype, key_at(slot / page_size, kvh, slot % page_size, da, n_kv_heads, page_size, head_dim), a);
                    store(k_cache, dtype, key_at(slot / page_size, kvh, slot % page_size, db, n_kv_heads, page_size, head_dim), b);
                } else {
                    int kvh = head - n_heads - n_kv_heads;
                    store(v_cache, dtype, value_at(slot / page_size, kvh, slot % page_size, da, n_kv_heads, page_size, head_dim), a);
                    store(v_cache, dtype, value_at(slot / page_size, kvh, slot % page_size, db, n_kv_heads, page_size, head_dim), b);
                }
            }
        }
    return 0;
}

// qkv = x W^T for W = [q heads; k heads; v heads] (a norm left to it applied as in llmrs_plain_gemm), q and k rotated
// by neighbouring pairs (2i, 2i+1) on the unrounded sums, q into `qkv`, k and v into the cache.  Only q's columns
// of `qkv` are written.
extern "C" int llmrs_plain_qkv_rope_cache(void*, int dtype, const void* x, int lda, const void* w, void* qkv, int row_stride,
                                          int M, int K, const int* positions, const int* slot_map, const float* inv_freq,
                                          int rotary_dim, void* k_cache, void* v_cache, int n_heads, int n_kv_heads,
                                          int head_dim, int page_size, int num_pages, int write_kv, void*, size_t, int,
                                          const float* scale_sumsq, int scale_parts, float scale_eps) {
    if (!known(dtype) || head_dim % 2 || rotary_dim % 2 || rotary_dim > head_dim || rotary_dim < 0) return -1;
    int heads = n_heads + 2 * n_kv_heads;
    std::vector<double> row(head_dim);
    for (int m = 0; m < M; ++m) {
        double inv = 1.0;
        if (scale_sumsq != nullptr) {
            double ss = 0.0;
            for (int p = 0; p < scale_parts; ++p) ss += scale_sumsq[(size_t)m * scale_parts + p];
            inv = 1.0 / std::sqrt(ss / K + (double)scale_eps);
        }
        for (int head = 0; head < heads; ++head) {
            bool is_q = head < n_heads, is_k = !is_q && head < n_heads + n_kv_heads;
            if (!is_q && !write_kv) continue;
            for (int d = 0; d < head_dim; ++d) {
                double s = 0.0;
                size_t n = (size_t)head * head_dim + d;
                for (int k = 0; k < K; ++k) s += load(x, dtype, (size_t)m * lda + k) * load(w, dtype, n * K + k);
                row[d] = s * inv;
            }
            if (is_q || is_k)
                for (int i = 0; i < rotary_dim / 2; ++i) {
                    double angle = (double)((float)positions[m] * inv_freq[i]);
                    double c = std::cos(angle), s = std::sin(angle);
                    double a = row[2 * i], b = row[2 * i + 1];
                    row[2 * i] = a * c - b * s;
                    row[2 * i + 1] = a * s + b * c;
                }
            if (is_q) {
                for (int d = 0; d < head_dim; ++d) store(qkv, dtype, (size_t)m * row_stride + (size_t)head * head_dim + d, row[d]);
                continue;
            }
            int slot = slot_map[m];
            if (slot < 0 || slot >= num_pages * page_size) continue;
            int page = slot / page_size, off = slot % page_size;
            for (int d = 0; d < head_dim; ++d) {
                if (is_k) store(k_cache, dtype, key_at(page, head - n_heads, off, d, n_kv_heads, page_size, head_dim), row[d]);
                else store(v_cache, dtype, value_at(page, head - n_heads - n_kv_heads, off, d, n_kv_heads, page_size, head_dim), row[d]);
            }
        }
    }
    return 0;
}

// For every query token t of entry e = token_entry[t] at position p = positions[t], every head: softmax over the keys
// max(0, p + 1 - window) .. p (all of 0 .. p without a window) of scale * q.k, times the values; key j of an entry
// lies in page block_table[e, j / page_size], slot j % page_size.  Heads share kv heads in groups of
// n_heads / n_kv_heads.
extern "C" int llmrs_plain_attention(void*, int dtype, const void* q, int q_stride, void* out, int out_stride,
                                     const void* k_cache, const void* v_cache, const int* block_table, int table_width,
                                     const int* token_entry, const int* positions, const int*, const int*, int n_entries,
                                     int n_tokens, int n_heads, int n_kv_heads, int head_dim, int page_size, int num_pages,
                                     int window, float scale, void*, size_t, int, int, long, int) {
    if (!known(dtype) || n_kv_heads <= 0 || n_heads % n_kv_heads || head_dim <= 0 || page_size <= 0) return -1;
    int group = n_heads / n_kv_heads;
    std::vector<double> score, acc(head_dim);
    for (int t = 0; t < n_tokens; ++t) {
        int e = token_entry[t], p = positions[t];
        if (e < 0 || e >= n_entries || p < 0 || p / page_size >= table_width) return -1;
        int lo = (window > 0 && p + 1 > window) ? p + 1 - window : 0;
        for (int h = 0; h < n_heads; ++h) {
            int kvh = h / group;
            score.assign(p + 1 - lo, 0.0);
            double top = -INFINITY;
            for (int j = lo; j <= p; ++j) {
                int page = block_table[(size_t)e * table_width + j / page_size];
                if (page < 0 || page >= num_pages) return -1;
                double dot = 0.0;
                for (int d = 0; d < head_dim; ++d)
                    dot += load(q, dtype, (size_t)t * q_stride + (size_t)h * head_dim + d) *
                           load(k_cache, dtype, key_at(page, kvh, j % page_size, d, n_kv_heads, page_size, head_dim));
                score[j - lo] = dot * (double)scale;
                top = std::max(top, score[j - lo]);
            }
            double total = 0.0;
            std::fill(acc.begin(), acc.end(), 0.0);
            for (int j = lo; j <= p; ++j) {
                double w = std::exp(score[j - lo] - top);
                total += w;
                int page = block_table[(size_t)e * table_width + j / page_size];
                for (int d = 0; d < head_dim; ++d)
                    acc[d] += w * load(v_cache, dtype, value_at(page, kvh, j % page_size, d, n_kv_heads, page_size, head_dim));
            }
            for (int d = 0; d < head_dim; ++d) store(out, dtype, (size_t)t * out_stride + (size_t)h * head_dim + d, acc[d] / total);
        }
    }
    return 0;
}

// The index of each row's largest value, the lowest such index.
extern "C" int llmrs_plain_argmax_rows(void*, const float* logits, int ld, int n_rows, int V, int* out, void*, size_t) {
    if (n_rows < 0 || V <= 0 || ld < V) return -1;
    for (int r = 0; r < n_rows; ++r) {
        const float* row = logits + (size_t)r * ld;
        int best = 0;
        for (int v = 1; v < V; ++v)
            if (row[v] > row[best]) best = v;
        out[r] = best;
    }
    return 0;
}

// tokens[rows[i]] = ids[sources[i]]; a pair outside either array, or an id outside the vocabulary, changes nothing.
extern "C" int llmrs_plain_place_ids(void*, int* tokens, int n_tokens, const int* rows, const int* sources, const int* ids,
                                     int n_ids, int n, int V) {
    if (n < 0 || n_tokens < 0 || n_ids < 0 || V <= 0) return -1;
    for (int i = 0; i < n; ++i) {
        if (rows[i] < 0 || rows[i] >= n_tokens || sources[i] < 0 || sources[i] >= n_ids) continue;
        int id = ids[sources[i]];
        if (id >= 0 && id < V) tokens[rows[i]] = id;
    }
    return 0;
}

namespace {
// The probabilities a row is drawn from (src/sampler/mod.rs:84-141): logits / temperature; all but the top_k largest
// dropped; softmax; the shortest prefix of the descending order whose mass reaches top_p kept and renormalised.  Of
// equal values at a cut the lowest indices stay.
void probabilities(const float* row, int V, float temperature, int top_k, float top_p, std::vector<double>& p) {
    std::vector<double> z(V);
    for (int v = 0; v < V; ++v) z[v] = (double)(row[v] * (1.0f / temperature));     // the scaled logit is a 32-bit product
    std::vector<int> order(V);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return z[a] > z[b]; });
    std::vector<char> kept(V, 1);
    if (top_k > 0 && top_k < V)
        for (int i = top_k; i < V; ++i) kept[order[i]] = 0;
    double top = z[order[0]], total = 0.0;
    p.assign(V, 0.0);
    for (int v = 0; v < V; ++v)
        if (kept[v]) { p[v] = std::exp(z[v] - top); total += p[v]; }
    for (int v = 0; v < V; ++v) p[v] /= total;
    if (top_p < 1.0f) {
        double cum = 0.0;
        int cutoff = V;
        for (int i = 0; i < V; ++i) {
            cum += p[order[i]];
            if (cum >= (double)top_p) { cutoff = i + 1; break; }
        }
        for (int i = cutoff; i < V; ++i) p[order[i]] = 0.0;
        double rest = 0.0;
        for (int v = 0; v < V; ++v) rest += p[v];
        if (rest > 0.0)
            for (int v = 0; v < V; ++v) p[v] /= rest;
    }
}
}  // namespace

// words: [n_rows, 4] = uniform (float bits), temperature (float bits), top_k, top_p (float bits).  A row with
// temperature 0 takes its largest logit; any other the first index, in index order, whose cumulative probability
// exceeds the uniform (src/sampler/mod.rs:143-154), the last kept index if rounding leaves none.
// probs (may be null): [n_rows, V], the probabilities each row was drawn from (a greedy row: 1 at its token).
extern "C" int llmrs_plain_sample_rows(void*, const float* logits, int ld, int n_rows, int V, const int* words, int* out,
                                       double* probs) {
    if (n_rows < 0 || V <= 0 || ld < V) return -1;
    std::vector<double> p;
    for (int r = 0; r < n_rows; ++r) {
        const float* row = logits + (size_t)r * ld;
        float u = bits_to_float(words[4 * r]), temperature = bits_to_float(words[4 * r + 1]), top_p = bits_to_float(words[4 * r + 3]);
        int top_k = words[4 * r + 2];
        if (!(temperature > 0.0f)) {
            llmrs_plain_argmax_rows(nullptr, row, ld, 1, V, out + r, nullptr, 0);
            if (probs != nullptr)
                for (int v = 0; v < V; ++v) probs[(size_t)r * V + v] = v == out[r] ? 1.0 : 0.0;
            continue;
        }
        probabilities(row, V, temperature, top_k, top_p, p);
        double cum = 0.0;
        int pick = -1, last = 0;
        for (int v = 0; v < V; ++v) {
            if (p[v] > 0.0) last = v;
            cum += p[v];
            if (pick < 0 && (double)u < cum) pick = v;
        }
        out[r] = pick >= 0 ? pick : last;
        if (probs != nullptr) std::copy(p.begin(), p.end(), probs + (size_t)r * V);
    }
    return 0;
}

// dst = src in dst's type: 0 float32, 1 bfloat16, and 2 float16 as a source only
extern "C" int llmrs_plain_cast(void*, void* dst, int dst_dtype, const void* src, int src_dtype, size_t n) {
    if (!known(dst_dtype) || src_dtype < 0 || src_dtype > 2) return -1;
    for (size_t i = 0; i < n; ++i) {
        double v;
        if (src_dtype == 2) {
            uint16_t hbits = ((const uint16_t*)src)[i];
            int sign = hbits >> 15, ex = (hbits >> 10) & 31, man = hbits & 1023;
            if (ex == 0) v = std::ldexp((double)man, -24);
            else if (ex == 31) v = man ? NAN : INFINITY;
            else v = std::ldexp((double)(man + 1024), ex - 25);
            if (sign) v = -v;
        } else {
            v = load(src, src_dtype, i);
        }
        store(dst, dst_dtype, i, v);
    }
    return 0;
}

// logits[r, v] <- logits[r, v] * scale, then, if cap > 0, cap * tanh(that / cap)
extern "C" int llmrs_plain_scale_softcap_rows(void*, float* logits, int ld, int n_rows, int V, float scale, float cap) {
    if (n_rows < 0 || V <= 0 || ld < V || cap < 0.0f) return -1;
    for (int r = 0; r < n_rows; ++r)
        for (int v = 0; v < V; ++v) {
            double x = (double)logits[(size_t)r * ld + v] * (double)scale;
            logits[(size_t)r * ld + v] = (float)(cap > 0.0f ? (double)cap * std::tanh(x / (double)cap) : x);
        }
    return 0;
}
