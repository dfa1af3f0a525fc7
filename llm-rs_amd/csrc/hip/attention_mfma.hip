// Paged causal attention on the matrix cores: bfloat16, pages of 16 slots,
// head sizes that are multiples of 32, up to 32 query heads per kv head.
//
// A wave owns a tile of 32 "query columns": the heads of one kv group for as many
// consecutive tokens of a request as fit (8 tokens x 4 heads for a 4:1 group; one
// token's heads when decoding).  It walks the request's keys 32 at a time:
//
//   S^T[key, col] = sum_d K[key, d] Q[col, d]      v_mfma_f32_32x32x16_bf16, A = K rows
//   online softmax down each column: a column is one lane pair, so the running
//   maximum and sum need one exchange with lane ^ 32 and no LDS
//   O^T[d, col]  += sum_key V^T[d, key] P^T[key, col]    A = V^T rows, B = P^T
//
// The accumulator of the first product is already the B operand of the second,
// if row r of the K operand holds key (r with bits 2 and 3 swapped): then lane
// half h holds, in registers 8s..8s+7, the probabilities of keys 16s + 8h + 0..7,
// which are the 8 consecutive slots of page s that the V^T operand reads with one
// 16-byte load (values lie [head_dim][slot] in a page).  No transpose, no LDS.
//
// Requests that bring one token (decoding) are split over waves by key range
// (ATTN_CHUNK keys or, with many requests, a multiple; aligned to absolute positions)
// and merged in ascending order by a second kernel.
//
// Math as in the reference's paged_attention (shaders/ops.metal:636-758): scale
// after the dot, mask = loop bound, max/exp/sums in 32-bit (the exponential as
// 2^(x log2 e), one instruction).  Probabilities are rounded to bfloat16 for the
// second product; their sum is not.
#include "attention.h"

#include <algorithm>
#include <cmath>
#include <mutex>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define ATTN_CHUNK 128


// all of this wave's vector memory operations, loads into LDS among them, have completed
__device__ __forceinline__ void wait_vmcnt_all() { __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8)); }
// all but the last N_ of them have completed (they complete in order)
template <int N_>
__device__ __forceinline__ void wait_vmcnt_n() {
    static_assert(N_ >= 0 && N_ < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N_ & 15) | (7 << 4) | (15 << 8) | ((N_ >> 4) << 14));
}

// The maximum (or sum) of a value over a lane and its partner in the other half of the wave,
// by the register swap of gfx950 (no trip through LDS).
__device__ __forceinline__ float other_half(float x) {
    unsigned u = __float_as_uint(x);
    auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);   // {x of the low half, x of the high half} in every lane
    return __uint_as_float((threadIdx.x & 32) ? sw[0] : sw[1]);
}

// The softmax step of one 32-key tile for this lane's column.  S holds the raw dots of the
// lane's 16 keys; on return it holds their probabilities relative to the reference value m
// (not yet normalised), m and l are updated, alpha is what the older sums must be scaled by.
// Scores are kept in the base-2 domain, (q.k) * c with c = scale * log2(e) > 0, so that the
// exponential is one v_exp_f32 of one fused multiply-add; the maximum is taken over the raw dots
// (c > 0 keeps the order).  Max, sums and scale factors are 32-bit as everywhere.
// m is a reference, not always the maximum: it follows the running maximum only when some
// column of the wave has outgrown it by more than 8 (a factor 256, far from the range's end in
// 32-bit sums and in the probabilities' bfloat16), which happens in the first tiles and then
// hardly ever.  Each column moves by its own rule, so its result does not depend on which
// other columns share its wave; whether any column moved is one answer for the wave (the
// return value: only then the older sums need scaling, by alpha, which is 1 in the columns
// that stayed).  The result is the same softmax: every term and the sum carry the same
// factor 2^(max - m).
// Keys outside [lo, pos] are masked; that pass is skipped (edge false, the same in all lanes)
// for tiles that lie wholly inside every column's range.
#define SOFTMAX_SLACK 8.0f
#define ATTN_WIDE_FROM_KEYS 32768        // tiles of eight waves from this bound on the step's lengths
__device__ __forceinline__ bool softmax_tile(f32x16& S, float& m, float& l, int t0, int pos, int lo,
                                             int h, float c, float& alpha, bool edge) {
    if (edge) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int key = t0 + 16 * (i >> 3) + 8 * h + 4 * ((i >> 2) & 1) + (i & 3);
            S[i] = (key > pos || key < lo) ? -INFINITY : S[i];
        }
    }
    float mx = S[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, S[i]);
    mx = fmaxf(mx, other_half(mx)) * c;
    bool mine = mx > m + SOFTMAX_SLACK;               // (-inf + 8 is -inf: a column's first key always moves it)
    bool move = __any(mine);
    alpha = 1.0f;
    if (__builtin_expect(move, 0)) {
        float m_new = mine ? mx : m;                  // each column by its own rule: nothing depends on its neighbours
        alpha = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.0f : m_new));
        m = m_new;
    }
    float m_safe = m == -INFINITY ? 0.0f : m;
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        S[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[i], c, -m_safe));
        sum += S[i];
    }
    sum += other_half(sum);
    l = l * alpha + sum;
    return move;
}

// One wave: keys [t_begin, t_end) (t_begin a multiple of 32) against its 32 columns.
// pos / lo: this lane's column may see keys lo..pos (pos < 0: nothing).
// The request's page numbers are fetched 64 at a time, one in each lane, so that a tile's keys
// need one trip to memory, not two in a row (page number, then keys).
template <int HD>
__device__ __forceinline__ void attend_range(const bf16x8 (&qf)[HD / 16], f32x16 (&O)[HD / 32], float& m, float& l,
                                             const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                                             const int* __restrict__ table, int table_width, int num_pages,
                                             int n_kv, int kvh, int t_begin, int t_end, int pos, int lo, float scale,
                                             bool have_pages = false, int first_pages = 0) {
    int lane = threadIdx.x & 63;
    int r = lane & 31, h = lane >> 5;
    float scale_log2e = scale * 1.44269504088896341f;
    float alpha_out;
    int kk = (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1);   // the key (within the tile) that K-operand row r holds
    if (t_begin >= t_end) return;
    int pv_base = t_begin >> 4;
    auto load_pages = [&](int first) {
        int pg = table[min(first + lane, table_width - 1)];
        return min(max(pg, 0), num_pages - 1);
    };
    int pv = have_pages ? first_pages : load_pages(pv_base);     // (the caller's: those of pages t_begin / 16 + lane, clamped as here)
    // Small heads leave registers for a second set of key operands: the next tile's keys are asked for before this
    // tile's products, one trip to memory per tile instead of two in a row (keys, then values).  At head size 128
    // that set would push the wave past 256 registers.
    constexpr bool KEYS_AHEAD = HD <= 64;
    int p0 = 0, p1 = 0;
    auto pages_of = [&](int t0, int& a0, int& a1) {
        int lp = t0 >> 4;
        if (lp + 1 - pv_base >= 64) { pv_base = lp; pv = load_pages(lp); }
        a0 = __builtin_amdgcn_readlane(pv, lp - pv_base);
        a1 = (t0 + 16 < t_end) ? __builtin_amdgcn_readlane(pv, lp + 1 - pv_base) : a0;   // a tile's second page may lie past the last key
    };
    auto keys_at = [&](int a0, int a1) { return kc + (((size_t)(kk < 16 ? a0 : a1) * n_kv + kvh) * 16 + (kk & 15)) * HD + h * 8; };
    bf16x8 kf[HD / 16];
    if constexpr (KEYS_AHEAD) {
        pages_of(t_begin, p0, p1);
        const bf16* kp = keys_at(p0, p1);
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) kf[ks] = *(const bf16x8*)(kp + ks * 16);
    }
    for (int t0 = t_begin; t0 < t_end; t0 += 32) {
        f32x16 S;
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] = 0.0f;
        int n0 = 0, n1 = 0;
        if constexpr (KEYS_AHEAD) {
            bf16x8 kn[HD / 16];
            const bool more = t0 + 32 < t_end;                   // (the same in all lanes)
            if (more) {
                pages_of(t0 + 32, n0, n1);
                const bf16* kp = keys_at(n0, n1);
#pragma unroll
                for (int ks = 0; ks < HD / 16; ++ks) kn[ks] = *(const bf16x8*)(kp + ks * 16);
            }
#pragma unroll
            for (int ks = 0; ks < HD / 16; ++ks) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], S, 0, 0, 0);
            if (more) {
#pragma unroll
                for (int ks = 0; ks < HD / 16; ++ks) kf[ks] = kn[ks];
            }
        } else {
            pages_of(t0, p0, p1);
            const bf16* kp = keys_at(p0, p1);
#pragma unroll
            for (int ks = 0; ks < HD / 16; ++ks) {
                bf16x8 k1 = *(const bf16x8*)(kp + ks * 16);
                S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k1, qf[ks], S, 0, 0, 0);
            }
        }
        // values of both pages: issued here so that their latency hides behind the softmax
        bf16x8 vf[HD / 32][2];
        const bf16* vp0 = vc + (((size_t)p0 * n_kv + kvh) * HD + r) * 16 + h * 8;
        const bf16* vp1 = vc + (((size_t)p1 * n_kv + kvh) * HD + r) * 16 + h * 8;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
            vf[dt][0] = *(const bf16x8*)(vp0 + dt * 32 * 16);
            vf[dt][1] = *(const bf16x8*)(vp1 + dt * 32 * 16);
        }
        bool moved = softmax_tile(S, m, l, t0, pos, lo, h, scale_log2e, alpha_out, __any(t0 + 31 > pos || t0 < lo));
        float alpha = alpha_out;
        bf16x8 pf[2];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pf[0][i] = (bf16)S[i];
            pf[1][i] = (bf16)S[8 + i];
        }
        if (moved) {                             // the reference rarely moves after the first tiles
#pragma unroll
            for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) O[dt][i] *= alpha;
        }
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
            O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][0], pf[0], O[dt], 0, 0, 0);
            O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][1], pf[1], O[dt], 0, 0, 0);
        }
        if constexpr (KEYS_AHEAD) { p0 = n0; p1 = n1; }
    }
}

// Feature that register i of O^T tile dt holds in lane half h.
__device__ __forceinline__ int o_feature(int dt, int i, int h) { return dt * 32 + 8 * (i >> 2) + 4 * h + (i & 3); }

// ---- entries with several tokens (and, when nothing is split, all entries) --
template <int HD>
__global__ __launch_bounds__(256) void attn_tiles_kernel(const bf16* __restrict__ q, bf16* __restrict__ out,
                                                         const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                                                         const int* __restrict__ block_table,
                                                         const int* __restrict__ positions,
                                                         const int* __restrict__ q_starts, int n_entries,
                                                         AttnArgs a, int G, int tpt, int skip_single) {
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int c = lane & 31, h = lane >> 5;
    int task = blockIdx.x * 4 + wave;
    int kvh = (task >> 2) % a.n_kv_heads;
    int tile = (task / (4 * a.n_kv_heads)) * 4 + (task & 3);
    int e = 0, rem = 0;
    if (!locate_tile(q_starts, n_entries, tpt, skip_single, tile, e, rem)) return;
    int tok0 = q_starts[e] + rem * tpt;
    int ntok = min(tpt, q_starts[e + 1] - tok0);
    int tq = c / G, hg = c - tq * G;
    bool cvalid = tq < ntok;
    int token = tok0 + min(tq, ntok - 1);
    int head = kvh * G + hg;
    int pos = cvalid ? positions[token] : -1;
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    int last = positions[tok0 + ntok - 1], first = positions[tok0];
    int t_end = last + 1;
    int t_begin = ((a.window > 0 && first + 1 > a.window) ? first + 1 - a.window : 0) & ~31;

    bf16x8 qf[HD / 16];
    const bf16* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + h * 8;
#pragma unroll
    for (int ks = 0; ks < HD / 16; ++ks) qf[ks] = *(const bf16x8*)(qp + ks * 16);
    f32x16 O[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    attend_range<HD>(qf, O, m, l, kc, vc, block_table + (size_t)e * a.table_width, a.table_width, a.num_pages,
                     a.n_kv_heads, kvh, t_begin, t_end, pos, lo, a.scale);
    if (!cvalid) return;
    float inv = 1.0f / l;
    bf16* op = out + (size_t)token * a.out_stride + (size_t)head * HD;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            bf16x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (bf16)(O[dt][i4 * 4 + j] * inv);
            *(bf16x4*)(op + o_feature(dt, i4 * 4, h)) = v;
        }
}

// ---- the same for head sizes 64, 128, 256, with the four waves of a block sharing their keys --
// The block's waves own four consecutive groups of tokens of one request and one kv head, so they
// want the same keys and values (up to the causal edge; every wave walks all of the block's
// tiles, those beyond its own keys masked).  Each 32-key tile (two pages of keys, two of values)
// is brought into LDS once, by global_load_lds straight from the cache's pages, several tiles
// ahead of its use (a ring of R tiles of keys and one of values); all four waves read their
// MFMA operands from there.  A key's row
// is 2*HD bytes and the rows lie unpadded, so chunk c of key kk is kept in slot c ^ swz(kk)
// (swz: kk for 256-byte rows and longer, kk >> 1 for 128-byte rows): the 16 lanes of an operand
// read want one chunk of 16 different keys and then hit 16 different bank groups.  Values are
// [HD][16] per page and are read in lane order; they need no swizzle.
template <int HD, int WAVES = 4>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(HD <= 128 ? 2 : 1))) void attn_tiles_lds_kernel(const bf16* __restrict__ q, bf16* __restrict__ out,
                                                             const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                                                             const int* __restrict__ block_table,
                                                             const int* __restrict__ positions,
                                                             const int* __restrict__ q_starts, int n_entries,
                                                             AttnArgs a, int G, int tpt, int skip_single,
                                                             int round_blocks) {
    constexpr int CHUNKS = HD / 8;                  // 16-byte chunks in a key's row
    constexpr int ROW_BYTES = HD * 2;
    constexpr int PAGE_BYTES = 16 * ROW_BYTES;      // a page of one kv head: keys [16][HD], values [HD][16]
    constexpr int TILE_BYTES = 2 * PAGE_BYTES;      // a tile's keys, or its values: two pages
    static_assert(WAVES == 4 || WAVES == 8, "four waves, or eight for long caches");
    constexpr int SHARE = PAGE_BYTES / (WAVES / 2); // bytes of a page that one wave brings: two pages, WAVES / 2 waves each
    static_assert(SHARE >= 1024 && SHARE % 1024 == 0, "a load instruction of a wave brings 1 KB");
    constexpr int HALF = SHARE / 1024;              // load instructions of a wave for its share of a page
    constexpr int SWZ_SHIFT = ROW_BYTES >= 256 ? 0 : 1;
    constexpr int R = (8 * TILE_BYTES <= 65536) ? 4 : 2;   // tiles in each of the two rings (keys, values)
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * R * TILE_BYTES];
    int lane = threadIdx.x & 63;
    int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // the same in all lanes: say so
    int c = lane & 31, h = lane >> 5;
    int kvh = blockIdx.x % a.n_kv_heads;
    // Order of work.  A tile's work grows with its place in its entry, so the tiles are handed out
    // from the last to the first: the longest start first, they decide when the grid ends.  All
    // blocks of the first two rounds (a round: as many blocks as the device holds at once in one
    // layer, `round_blocks`) are resident together, the second round beside the first on the same
    // units, so the second round runs in the opposite order and puts the shortest beside the longest
    // (`round_blocks` 0, for blocks that have a unit to themselves: from the last to the first throughout).
    int n_btiles = count_tiles(q_starts, n_entries, WAVES * tpt, skip_single);      // (every wave for itself: the same figures)
    int g = blockIdx.x / a.n_kv_heads;
    if (g >= n_btiles) return;                       // the grid is sized for the most tiles the tokens could make
    int gr = round_blocks / a.n_kv_heads;
    if (g >= gr && g < 2 * gr) g = gr + (min(2 * gr, n_btiles) - 1 - g);
    int btile = n_btiles - 1 - g;                    // WAVES * tpt tokens of one entry
    int e = 0, rem = 0;
    if (!locate_tile(q_starts, n_entries, WAVES * tpt, skip_single, btile, e, rem)) return;
    int e_end = q_starts[e + 1];
    int btok0 = q_starts[e] + rem * WAVES * tpt;
    int btok_last = min(btok0 + WAVES * tpt, e_end) - 1;
    // this wave's tokens (it may have none, at the end of an entry: it still helps to load)
    int tok0 = btok0 + wave * tpt;
    int ntok = max(0, min(tpt, e_end - tok0));
    bool wave_active = ntok > 0;
    int tq = c / G, hg = c - tq * G;
    bool cvalid = tq < ntok;
    int token = wave_active ? tok0 + min(tq, ntok - 1) : btok0;
    int head = kvh * G + hg;
    int pos = cvalid ? positions[token] : -1;
    int lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    // An entry's positions rise by one from token to token, so the first and last token bound the rest.
    int b_first = positions[btok0], b_last = positions[btok_last];
    int t_end = b_last + 1;                                          // keys the block needs: [t_begin, t_end)
    int t_begin = ((a.window > 0 && b_first + 1 > a.window) ? b_first + 1 - a.window : 0) & ~31;
    int w_first = wave_active ? positions[tok0] : 0;                 // this wave's first and last position
    int w_last = wave_active ? positions[tok0 + ntok - 1] : -1;
    int w_lo_last = (a.window > 0 && w_last + 1 > a.window) ? w_last + 1 - a.window : 0;
    const int* table = block_table + (size_t)e * a.table_width;

    bf16x8 qf[HD / 16];
    const bf16* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + h * 8;
#pragma unroll
    for (int ks = 0; ks < HD / 16; ++ks) qf[ks] = *(const bf16x8*)(qp + ks * 16);
    f32x16 O[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    float scale_log2e = a.scale * 1.44269504088896341f;

    // ---- loads.  A tile's keys are two pages and so are its values; each wave brings its share of a
    // page of both (page wave & 1, share wave >> 1: half a page with four waves, a quarter with eight).  What a lane fetches for its place in the page's
    // LDS image does not change from tile to tile:
    unsigned goff_k[HALF], goff_v[HALF];
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
        int off = (wave >> 1) * SHARE + i * 1024 + lane * 16;
        int krow = off / ROW_BYTES, slot = (off % ROW_BYTES) / 16;
        goff_k[i] = krow * ROW_BYTES + ((slot ^ ((krow >> SWZ_SHIFT) & (CHUNKS - 1) & 15)) * 16);   // keys: the chunk that belongs in this slot
        goff_v[i] = off;
    }
    unsigned lds_part = (wave & 1) * PAGE_BYTES + (wave >> 1) * SHARE;   // this wave's part of a tile's image
    const unsigned char* k_base = (const unsigned char*)(kc + (size_t)kvh * (16 * HD));
    const unsigned char* v_base = (const unsigned char*)(vc + (size_t)kvh * (16 * HD));
    size_t page_stride = (size_t)a.n_kv_heads * (16 * HD) * sizeof(bf16);
    int n = (t_end - t_begin + 31) >> 5;             // tiles of the block, numbered from 0
    int lp0 = t_begin >> 4;                          // the first tile's first logical page
    // The request's page numbers for 64 logical pages at a time, one in each lane.
    int pv_base = lp0;
    auto load_pages = [&](int first) {
        int pg = table[min(first + lane, a.table_width - 1)];
        return min(max(pg, 0), a.num_pages - 1);
    };
    int pv = load_pages(pv_base);
    // Everything read from memory so far (the queries above all) is waited for here, once: a wait
    // for it inside the loop would be a wait for all of the loop's own loads each time round.
    wait_vmcnt_all();
    auto page_of = [&](int tile) {                   // the page this wave loads from, for a tile in [0, n)
        int lp = lp0 + 2 * tile;
        // a tile's second page may lie past the request's last key: then it is not looked up
        int idx = lp - pv_base + (((wave & 1) && t_begin + 32 * tile + 16 < t_end) ? 1 : 0);
        return (size_t)__builtin_amdgcn_readlane(pv, idx) * page_stride;
    };
    auto load_part = [&](const unsigned char* src, const unsigned (&goff)[HALF], int lds_off) {
#pragma unroll
        for (int i = 0; i < HALF; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + goff[i]),
                                             (__attribute__((address_space(3))) void*)(lds + lds_off + lds_part + i * 1024),
                                             16, 0, 0);
    };
    // What iteration t starts on their way: keys of tile t + R (into the slot whose tile, t, went
    // into the products of iteration t - 1), values of tile t + R - 1 (tile t - 1 was used in
    // iteration t - 1).  `t mod R` is passed apart, as a constant.  Every iteration starts the
    // same number of loads: where the tile would lie outside [0, n) the nearest real one is
    // loaded once more, into a slot that nobody reads; that costs less than telling the cases apart.
    auto issue = [&](int t, int t_mod) {
        int tk = min(t + R, n - 1), tv = min(max(t + R - 1, 0), n - 1);
        if (__builtin_expect(lp0 + 2 * tk + 1 - pv_base >= 64, 0)) {      // tv <= tk: its pages stay in the window
            pv_base = lp0 + 2 * tv;
            pv = load_pages(pv_base);
        }
        load_part(k_base + page_of(tk), goff_k, ((t_mod + R) % R) * TILE_BYTES);
        load_part(v_base + page_of(tv), goff_v, (R + (t_mod + R - 1) % R) * TILE_BYTES);
    };
    // At the end of iteration t the keys of tile t + 2 and the values of tile t + 1 must have
    // landed: all that iteration t + 2 - R and those before it started.  Loads complete in order,
    // so the wave may leave behind what it has started since then.
    auto wait_landed = [&]() { wait_vmcnt_n<2 * (R - 2) * HALF>(); };
    // All waves are done with what they read from LDS (the reads have returned), and what each
    // waited for above is there for everybody.  A bare s_barrier: __syncthreads() would also wait
    // for the loads that are meant to stay in flight.
    auto block_sync = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    int r = lane & 31;
    int kk = (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1);   // the key (within the tile) that K-operand row r holds
    int kswz = ((kk & 15) >> SWZ_SHIFT) & (CHUNKS - 1) & 15;
    unsigned koffs[HD / 16];                                  // where this lane's K operands lie in a tile's image
#pragma unroll
    for (int ks = 0; ks < HD / 16; ++ks)
        koffs[ks] = (kk >> 4) * PAGE_BYTES + (kk & 15) * ROW_BYTES + (((ks * 2 + h) ^ kswz) * 16);
    unsigned voff = r * 32 + h * 16;

    // S^T of a tile from the keys in ring slot `slot`
    auto scores = [&](int slot) {
        const unsigned char* st = lds + slot * TILE_BYTES;
        bf16x8 kf[HD / 16];
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) kf[ks] = *(const bf16x8*)(st + koffs[ks]);
        f32x16 S;
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], S, 0, 0, 0);
        return S;
    };
    // The values in ring slot `slot` as operands, and O^T += V^T P^T with them.  The two are
    // apart so that the reads can be started before the softmax arithmetic and return behind it.
    constexpr int VF = HD / 32 * 2;
    auto read_values = [&](int slot, bf16x8 (&vf)[VF]) {
        const unsigned char* st = lds + (R + slot) * TILE_BYTES + voff;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
            vf[2 * dt] = *(const bf16x8*)(st + dt * 32 * 32);
            vf[2 * dt + 1] = *(const bf16x8*)(st + PAGE_BYTES + dt * 32 * 32);
        }
    };
    auto accumulate = [&](const bf16x8 (&vf)[VF], const bf16x8 (&pf)[2]) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
            O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[2 * dt], pf[0], O[dt], 0, 0, 0);
            O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[2 * dt + 1], pf[1], O[dt], 0, 0, 0);
        }
    };
    auto rescale = [&](bool moved, float alpha) {
        if (__builtin_expect(moved, 0)) {             // the reference rarely moves after the first tiles
#pragma unroll
            for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) O[dt][i] *= alpha;
        }
    };
    // some column of the wave has a key of tile t masked (tiles beyond a wave's own keys are
    // masked as a whole: every wave walks all of the block's tiles)
    auto is_edge = [&](int t) { int t0 = t_begin + 32 * t; return t0 + 31 > w_first || t0 < w_lo_last; };
    auto to_bf16 = [&](const f32x16& S, bf16x8 (&pf)[2]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pf[0][i] = (bf16)S[i];
            pf[1][i] = (bf16)S[8 + i];
        }
    };

    // The score products of a tile and the softmax arithmetic of the tile before do not depend on
    // each other, so the loop is skewed: iteration t starts the scores of tile t + 1 (matrix
    // cores) beside the softmax of tile t (vector unit), then adds tile t's values.
#pragma unroll
    for (int j = 0; j < R; ++j) issue(j - R, j);                    // keys 0 .. R-1, values 0 .. R-2
    wait_landed();                                                   // keys of tiles 0 and 1, values of tile 0
    block_sync();
    f32x16 S_next = scores(0);
    block_sync();                                                    // tile 0's keys may be overwritten
    for (int tb = 0; tb < n; tb += R) {
#pragma unroll
        for (int s = 0; s < R; ++s) {                 // unrolled: the ring slots are constants, LDS addresses immediates
            int t = tb + s;                           // t mod R == s
            if (t >= n) break;
            issue(t, s);
            f32x16 S_cur = S_next;
            float alpha;
            bf16x8 pf[2], vf[VF];
            bool moved;
            if (is_edge(t)) {
                S_next = scores((s + 1) % R);         // (nothing real for the last tile: not used then)
                read_values(s, vf);
                moved = softmax_tile(S_cur, m, l, t_begin + 32 * t, pos, lo, h, scale_log2e, alpha, true);
            } else {
                S_next = scores((s + 1) % R);
                read_values(s, vf);
                moved = softmax_tile(S_cur, m, l, t_begin + 32 * t, pos, lo, h, scale_log2e, alpha, false);
            }
            to_bf16(S_cur, pf);
            rescale(moved, alpha);
            accumulate(vf, pf);
            wait_landed();
            block_sync();
        }
    }

    if (!cvalid) return;
    float inv = 1.0f / l;
    bf16* op = out + (size_t)token * a.out_stride + (size_t)head * HD;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            bf16x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (bf16)(O[dt][i4 * 4 + j] * inv);
            *(bf16x4*)(op + o_feature(dt, i4 * 4, h)) = v;
        }
}

// ---- entries with one token: a wave for each (entry, kv head, chunk of keys) --
// partial: [(entry * n_heads + head) * max_chunks + chunk][HD + 2] = m, l, O (not yet divided)
// With `plain` (every entry brings one token and there is no window) a wave knows its token (the entry's number) and
// where its keys begin (ch * chunk) without the request's length: it asks for its page numbers and its queries together
// with the length, one trip to memory instead of two in a row.
template <int HD>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 3 : 1))) void attn_split_kernel(const bf16* __restrict__ q, float* __restrict__ partial,
                                                        const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                                                        const int* __restrict__ block_table,
                                                        const int* __restrict__ seq_lens,
                                                        const int* __restrict__ q_starts, AttnArgs a, int G,
                                                        int max_chunks, int chunk, int plain) {
    int e = blockIdx.x, kvh = blockIdx.y, ch = blockIdx.z;
    int lane = threadIdx.x & 63, c = lane & 31, h = lane >> 5;
    bool cvalid = c < G;
    int head = kvh * G + min(c, G - 1);
    const int* table = block_table + (size_t)e * a.table_width;
    bf16x8 qf[HD / 16];
    int token, pos_t, lo_t, t_begin, first_pages = 0;
    if (plain) {
        token = e;
        lo_t = 0;
        t_begin = ch * chunk;
        int pg = table[min((t_begin >> 4) + lane, a.table_width - 1)];
        first_pages = min(max(pg, 0), a.num_pages - 1);
        const bf16* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + h * 8;
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) qf[ks] = *(const bf16x8*)(qp + ks * 16);
        pos_t = seq_lens[e] - 1;                  // an entry with one token: its position is its length less one
        if (t_begin > pos_t) return;
    } else {
        token = q_starts[e];
        int count = q_starts[e + 1] - token;
        pos_t = seq_lens[e] - 1;
        if (count != 1) return;
        lo_t = (a.window > 0 && pos_t + 1 > a.window) ? pos_t + 1 - a.window : 0;
        int first_chunk = lo_t / chunk;
        int n_chunks = pos_t / chunk - first_chunk + 1;
        if (ch >= n_chunks) return;
        t_begin = (first_chunk + ch) * chunk;
        const bf16* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + h * 8;
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) qf[ks] = *(const bf16x8*)(qp + ks * 16);
    }
    int t_end = min(t_begin + chunk, pos_t + 1);
    int pos = cvalid ? pos_t : -1;
    f32x16 O[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    attend_range<HD>(qf, O, m, l, kc, vc, table, a.table_width, a.num_pages,
                     a.n_kv_heads, kvh, t_begin, t_end, pos, lo_t, a.scale, plain != 0, first_pages);
    if (!cvalid) return;
    float* pp = partial + ((size_t)(e * a.n_heads + head) * max_chunks + ch) * (HD + 2);
    if (h == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) pp[2 + o_feature(dt, i, h)] = O[dt][i];
}

// ---- the same with 16 query columns to a wave (up to 16 heads to a kv head) --
// A single token brings G query columns; the 32-column products above spend their accumulators on 32 - G columns
// of nothing.  Here S^T = K Q^T is two 16 x 16 tiles per 32 keys and O^T += V^T P^T one product per 16 features
// with the 32 keys as its k: a quarter of the accumulators and half of the exponentials, so that a SIMD holds
// more of these waves, and with them more keys on their way.
// Which keys a 16-row tile holds is free, as long as the values' operand takes them in the same order: tile t of a
// 32-key step holds key 8 * (row / 4) + row % 4 + 4 * t in its row, so lane (col, g) ends with the scores of keys
// 8g .. 8g + 7 in its eight registers (tile 0's four, then tile 1's): the B operand of the second product as it
// stands, and for the values, [feature][16 keys] per page, one 16-byte load per lane and 16 features.
typedef float f32x4 __attribute__((ext_vector_type(4)));
// The registers would let a SIMD hold three of these waves at head size 128 and four at 64, and with twelve or
// sixteen to a compute unit the scattered pages come slower than with eight once the device is full (decode steps
// of the 8B shape, eight waves against twelve: 64 requests over 8128 keys 15.9 against 16.9 ms, 256 over 2048 18.3
// against 20.7; the 1B serving run 3.03 against 3.10 s with sixteen).  Every block asks for an eighth of a
// unit's LDS, which it does not use, and that keeps a unit to eight.
#define SPLIT16_LDS_BYTES (160 * 1024 / 8)

// The value of the lane 16 further on or back (the partner in the neighbouring row of 16 lanes), by the register
// swap of gfx950: of {x, x} it makes {rows 0, 0, 2, 2 of x; rows 1, 1, 3, 3 of x}.
__device__ __forceinline__ float other_row(float x) {
    unsigned u = __float_as_uint(x);
    auto sw = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return __uint_as_float((threadIdx.x & 16) ? sw[0] : sw[1]);
}
__device__ __forceinline__ float across_groups_max(float x) {
    x = fmaxf(x, other_row(x));
    return fmaxf(x, other_half(x));
}
__device__ __forceinline__ float across_groups_sum(float x) {
    x += other_row(x);
    return x + other_half(x);
}

template <int HD>
__global__ __launch_bounds__(64) void attn_split16_kernel(const bf16* __restrict__ q, float* __restrict__ partial,
                                                          const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                                                          const int* __restrict__ block_table,
                                                          const int* __restrict__ seq_lens,
                                                          const int* __restrict__ q_starts, AttnArgs a, int G,
                                                          int max_chunks, int chunk, int plain) {
    static_assert(HD % 32 == 0, "the score products take 32 features at a time");
    int e = blockIdx.x, kvh = blockIdx.y, ch = blockIdx.z;
    int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
    bool cvalid = c < G;
    int head = kvh * G + min(c, G - 1);
    const int* table = block_table + (size_t)e * a.table_width;
    bf16x8 qf[HD / 32];
    int token, pos_t, lo_t, t_begin, pv = 0;
    auto load_pages = [&](int first) {
        int pg = table[min(first + lane, a.table_width - 1)];
        return min(max(pg, 0), a.num_pages - 1);
    };
    if (plain) {
        token = e;
        lo_t = 0;
        t_begin = ch * chunk;
        pv = load_pages(t_begin >> 4);
        const bf16* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + g * 8;
#pragma unroll
        for (int j = 0; j < HD / 32; ++j) qf[j] = *(const bf16x8*)(qp + j * 32);
        pos_t = seq_lens[e] - 1;
        if (t_begin > pos_t) return;
    } else {
        token = q_starts[e];
        int count = q_starts[e + 1] - token;
        pos_t = seq_lens[e] - 1;
        if (count != 1) return;
        lo_t = (a.window > 0 && pos_t + 1 > a.window) ? pos_t + 1 - a.window : 0;
        int first_chunk = lo_t / chunk;
        int n_chunks = pos_t / chunk - first_chunk + 1;
        if (ch >= n_chunks) return;
        t_begin = (first_chunk + ch) * chunk;
        pv = load_pages(t_begin >> 4);
        const bf16* qp = q + (size_t)token * a.q_stride + (size_t)head * HD + g * 8;
#pragma unroll
        for (int j = 0; j < HD / 32; ++j) qf[j] = *(const bf16x8*)(qp + j * 32);
    }
    int t_end = min(t_begin + chunk, pos_t + 1);
    int pv_base = t_begin >> 4;
    float c2 = a.scale * 1.44269504088896341f;
    f32x4 O[HD / 16];
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) O[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.0f;                    // m: the same in a column's four lanes; l: this lane's share of the sum
    // the keys of tile t that this lane's operand row holds, within a 32-key step: 8 * (row / 4) + row % 4 + 4t
    int krow = 8 * (c >> 2) + (c & 3);
    // A unit holds eight of these waves whatever they take (see SPLIT16_LDS_BYTES), so up to head size 128 a wave has
    // the registers for a second set of key operands: the next step's keys are asked for before this step's products.
    constexpr bool KEYS_AHEAD = HD <= 128;
    auto pages_of = [&](int t0, int& a0, int& a1) {
        int lp = t0 >> 4;
        if (lp + 1 - pv_base >= 64) { pv_base = lp; pv = load_pages(lp); }
        a0 = __builtin_amdgcn_readlane(pv, lp - pv_base);
        a1 = (t0 + 16 < t_end) ? __builtin_amdgcn_readlane(pv, lp + 1 - pv_base) : a0;
    };
    auto load_keys = [&](bf16x8 (&k)[2][HD / 32], int a0, int a1) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            int key = krow + 4 * t;                                   // 0..31: page key >> 4, row key & 15
            const bf16* kp = kc + (((size_t)(key < 16 ? a0 : a1) * a.n_kv_heads + kvh) * 16 + (key & 15)) * HD + g * 8;
#pragma unroll
            for (int j = 0; j < HD / 32; ++j) k[t][j] = *(const bf16x8*)(kp + j * 32);
        }
    };
    bf16x8 kf[2][HD / 32];
    int p0 = 0, p1 = 0;
    if constexpr (KEYS_AHEAD) {
        pages_of(t_begin, p0, p1);
        load_keys(kf, p0, p1);
    }
    for (int t0 = t_begin; t0 < t_end; t0 += 32) {
        bf16x8 kn[2][HD / 32];
        int n0 = 0, n1 = 0;
        const bool more = t0 + 32 < t_end;                            // (the same in all lanes)
        if constexpr (KEYS_AHEAD) {
            if (more) {
                pages_of(t0 + 32, n0, n1);
                load_keys(kn, n0, n1);
            }
        } else {
            pages_of(t0, p0, p1);
            load_keys(kf, p0, p1);
        }
        // values: lane (feature row c, g) takes keys 8g .. 8g + 7 of the step: page g / 2, keys 8 * (g % 2) .. of it
        bf16x8 vf[HD / 16];
        const bf16* vp = vc + (((size_t)(g < 2 ? p0 : p1) * a.n_kv_heads + kvh) * HD + c) * 16 + (g & 1) * 8;
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt) vf[dt] = *(const bf16x8*)(vp + dt * 16 * 16);
        f32x4 S[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            S[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < HD / 32; ++j) S[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][j], qf[j], S[t], 0, 0, 0);
        }
        // this lane's scores: keys t0 + 8g + i, i = 0..7 (tile 0's registers, then tile 1's)
        float sc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) sc[i] = S[i >> 2][i & 3];
        if (t0 + 31 > pos_t || t0 < lo_t) {                           // (the same in all lanes)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int key = t0 + 8 * g + i;
                if (key > pos_t || key < lo_t) sc[i] = -INFINITY;
            }
        }
        float mx = sc[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) mx = fmaxf(mx, sc[i]);
        mx = across_groups_max(mx) * c2;
        bool mine = mx > m + SOFTMAX_SLACK;
        if (__any(mine)) {
            float m_new = mine ? mx : m;
            float alpha = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.0f : m_new));
            m = m_new;
            l *= alpha;
#pragma unroll
            for (int dt = 0; dt < HD / 16; ++dt) O[dt] *= alpha;
        }
        float m_safe = m == -INFINITY ? 0.0f : m;
        bf16x8 pf;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], c2, -m_safe));
            l += p;
            pf[i] = (bf16)p;
        }
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt) O[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pf, O[dt], 0, 0, 0);
        if constexpr (KEYS_AHEAD) {
            if (more) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int j = 0; j < HD / 32; ++j) kf[t][j] = kn[t][j];
                p0 = n0; p1 = n1;
            }
        }
    }
    l = across_groups_sum(l);
    if (!cvalid) return;
    float* pp = partial + ((size_t)(e * a.n_heads + head) * max_chunks + ch) * (HD + 2);
    if (g == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) pp[2 + dt * 16 + 4 * g + r] = O[dt][r];
}

#define MERGE_MAX_CHUNKS 1024

// One block for each (entry, head), a thread for each feature (a wave per 64 of them).  Every wave finds the common
// maximum and the sum for itself, its lanes sharing out the chunks; chunks are added in ascending order.  Everything
// a thread needs from memory is asked for at once (a chunk's m and l, and its feature's sums for the first
// chunks): the kernel is a chain of trips to memory and little else.
// With `plain` (every entry brings one token, no window) the token is the entry's number and the chunks are
// counted from the first: the first chunks' sums, maxima and sums of weights are asked for before the
// request's length is known (what lies beyond its chunks is read and never used), one trip instead of two.
__global__ __launch_bounds__(256) void attn_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out,
                                                         const int* __restrict__ seq_lens,
                                                         const int* __restrict__ q_starts, AttnArgs a, int max_chunks,
                                                         int chunk, int plain) {
    __shared__ float weight[MERGE_MAX_CHUNKS];
    constexpr int AHEAD = 32;                     // chunks whose sums are asked for before the weights are known
    int e = blockIdx.x, head = blockIdx.y, hd = a.head_dim, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int d = threadIdx.x;                          // this thread's feature (threads past the head size only help with the weights)
    const float* pp = partial + (size_t)(e * a.n_heads + head) * max_chunks * (hd + 2);
    int stride = hd + 2;
    int token, pos, lo, n_chunks;
    float ahead[AHEAD];
    float m_mine = -INFINITY, l_mine = 0.0f;      // chunk `lane`'s maximum and sum (plain, up to 64 chunks)
    const bool early = plain && max_chunks <= 64;
    if (early) {
#pragma unroll
        for (int ch = 0; ch < AHEAD; ++ch) ahead[ch] = (ch < max_chunks && d < hd) ? pp[(size_t)ch * stride + 2 + d] : 0.0f;
        if (lane < max_chunks) { m_mine = pp[(size_t)lane * stride]; l_mine = pp[(size_t)lane * stride + 1]; }
        token = e;
        pos = seq_lens[e] - 1;
        lo = 0;
        n_chunks = pos / chunk + 1;
    } else {
        token = q_starts[e];
        int count = q_starts[e + 1] - token;
        pos = seq_lens[e] - 1;
        if (count != 1) return;
        lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
        n_chunks = pos / chunk - lo / chunk + 1;
#pragma unroll
        for (int ch = 0; ch < AHEAD; ++ch) ahead[ch] = (ch < n_chunks && d < hd) ? pp[(size_t)ch * stride + 2 + d] : 0.0f;
    }
    float M = -INFINITY;
    float L = 0.0f;
    if (early) {
        if (lane >= n_chunks) m_mine = -INFINITY;
        M = wave_max(m_mine);
        float w = lane < n_chunks ? __builtin_amdgcn_exp2f(m_mine - M) : 0.0f;     // the maxima are base-2 logarithms
        if (lane < n_chunks) { if (wave == 0) weight[lane] = w; L = l_mine * w; }
    } else {
        for (int ch = lane; ch < n_chunks; ch += 64) M = fmaxf(M, pp[(size_t)ch * stride]);
        M = wave_max(M);
        for (int ch = lane; ch < n_chunks; ch += 64) {
            float w = __builtin_amdgcn_exp2f(pp[(size_t)ch * stride] - M);
            if (wave == 0) weight[ch] = w;
            L += pp[(size_t)ch * stride + 1] * w;
        }
    }
    L = wave_sum(L);
    __syncthreads();
    if (d >= hd) return;
    float o = 0.0f;
#pragma unroll
    for (int c = 0; c < AHEAD; ++c)
        if (c < n_chunks) o = fmaf(ahead[c], weight[c], o);
    for (int ch = AHEAD; ch < n_chunks; ch += AHEAD) {      // the rest, a group's sums asked for together
        float v[AHEAD];
#pragma unroll
        for (int c = 0; c < AHEAD; ++c) v[c] = (ch + c < n_chunks) ? pp[(size_t)(ch + c) * stride + 2 + d] : 0.0f;
#pragma unroll
        for (int c = 0; c < AHEAD; ++c)
            if (ch + c < n_chunks) o = fmaf(v[c], weight[ch + c], o);
    }
    out[(size_t)token * a.out_stride + (size_t)head * hd + d] = (bf16)(o / L);
}

// The merge for more than a few chunks (131,000 keys of one request are 256 chunks of 512).  One thread per
// feature walks the chunks one after the other, 32 loads at a time, each batch a trip to memory: 45 us for 256
// chunks, where the split itself takes 97; 2.1 and 2.6 us a layer more than this kernel at 32 and 63 chunks (one
// request, 2048 and 4000 keys), the same at 16 (8 to 32 requests).  Here the block's threads stand in groups, each group a
// row of the partial sums wide (two features a thread), and the groups share out the chunks: with 16 loads asked
// for at once a block has 128 chunks' rows (256 at head size 64) in flight.  The groups' sums meet in LDS and are
// added in the order of the groups, so the result does not depend on timing.  Weights as in the kernel above.
#define MERGE_GROUP_THREADS 512
#define MERGE_ONE_WALK_CHUNKS 8       // up to here a thread per feature walks the chunks alone (many requests, short caches)
__global__ __launch_bounds__(MERGE_GROUP_THREADS) void attn_merge_groups_kernel(
        const float* __restrict__ partial, bf16* __restrict__ out, const int* __restrict__ seq_lens,
        const int* __restrict__ q_starts, AttnArgs a, int max_chunks, int chunk, int plain) {
    __shared__ float weight[MERGE_MAX_CHUNKS];
    __shared__ float sums[2 * MERGE_GROUP_THREADS];
    constexpr int AHEAD = 16;
    int e = blockIdx.x, head = blockIdx.y, hd = a.head_dim, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int per_row = hd / 2;                         // threads to a chunk's row (head sizes are even)
    int groups = blockDim.x / per_row;            // (the launch gives a group four chunks or more)
    int g = tid / per_row, f = tid - g * per_row; // threads past the last whole group only help with the weights
    const bool adds = g < groups;
    int stride = hd + 2;
    const float* pp = partial + (size_t)(e * a.n_heads + head) * max_chunks * stride;
    int token, pos, lo;
    if (plain) {
        token = e;
        pos = seq_lens[e] - 1;
        lo = 0;
    } else {
        token = q_starts[e];
        int count = q_starts[e + 1] - token;
        if (count != 1) return;                   // (the whole block: nothing below is reached by a part of it)
        pos = seq_lens[e] - 1;
        lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
    }
    int n_chunks = pos / chunk - lo / chunk + 1;
    const float* mine = pp + 2 + 2 * f;           // 8-byte aligned: rows of hd + 2 floats, hd even
    float2 ahead[AHEAD];
#pragma unroll
    for (int c = 0; c < AHEAD; ++c) {
        int ch = g + c * groups;
        ahead[c] = (adds && ch < n_chunks) ? *reinterpret_cast<const float2*>(mine + (size_t)ch * stride) : make_float2(0.0f, 0.0f);
    }
    float M = -INFINITY, L = 0.0f;
    for (int ch = lane; ch < n_chunks; ch += 64) M = fmaxf(M, pp[(size_t)ch * stride]);
    M = wave_max(M);
    for (int ch = lane; ch < n_chunks; ch += 64) {
        float w = __builtin_amdgcn_exp2f(pp[(size_t)ch * stride] - M);      // the maxima are base-2 logarithms
        if (wave == 0) weight[ch] = w;
        L += pp[(size_t)ch * stride + 1] * w;
    }
    L = wave_sum(L);
    __syncthreads();
    if (adds) {
        float ox = 0.0f, oy = 0.0f;
#pragma unroll
        for (int c = 0; c < AHEAD; ++c) {
            int ch = g + c * groups;
            if (ch < n_chunks) { float w = weight[ch]; ox = fmaf(ahead[c].x, w, ox); oy = fmaf(ahead[c].y, w, oy); }
        }
        for (int base = g + AHEAD * groups; base < n_chunks; base += AHEAD * groups) {
            float2 v[AHEAD];
#pragma unroll
            for (int c = 0; c < AHEAD; ++c) {
                int ch = base + c * groups;
                v[c] = ch < n_chunks ? *reinterpret_cast<const float2*>(mine + (size_t)ch * stride) : make_float2(0.0f, 0.0f);
            }
#pragma unroll
            for (int c = 0; c < AHEAD; ++c) {
                int ch = base + c * groups;
                if (ch < n_chunks) { float w = weight[ch]; ox = fmaf(v[c].x, w, ox); oy = fmaf(v[c].y, w, oy); }
            }
        }
        sums[g * hd + 2 * f] = ox;
        sums[g * hd + 2 * f + 1] = oy;
    }
    __syncthreads();
    if (tid < hd) {
        float o = 0.0f;
        for (int k = 0; k < groups; ++k) o += sums[k * hd + tid];
        out[(size_t)token * a.out_stride + (size_t)head * hd + tid] = (bf16)(o / L);
    }
}

// A step with a prompt portion beside decoding requests has two kinds of attention work that do not depend on
// each other: tiles of many tokens, bound by the matrix cores, and single tokens over their whole caches, bound by
// memory.  They run side by side: the single tokens' kernels go to a second stream of this library's own (default
// priority), which waits for everything the caller's stream held when the call came and which the caller's stream
// waits for before it goes on.  One such stream and pair of events per device, made at first use.  While the
// caller's stream is being captured into a graph nothing is forked: the two kinds follow each other as before.
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool tried = false;
};
static SideStream* side_stream() {
    static SideStream per_device[64];
    static std::mutex mutex;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> lock(mutex);
    SideStream& s = per_device[dev];
    if (!s.tried) {
        s.tried = true;
        bool ok = hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) == hipSuccess &&
                  hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) == hipSuccess &&
                  hipEventCreateWithFlags(&s.join, hipEventDisableTiming) == hipSuccess;
        if (!ok) { (void)hipGetLastError(); s.stream = nullptr; }
    }
    return s.stream != nullptr ? &s : nullptr;
}

// How many waves of the split a compute unit holds at once: eight (see SPLIT16_LDS_BYTES), fewer where the registers
// of the kernel for this head size allow no more (four at head size 256), asked of the runtime once per head size.
// Head sizes without a kernel here: 8.  (The 32-column kernel, for more than 16 heads to a kv head, holds eight at
// head size 128 as well and twelve at 64; its chunks are chosen as if it held eight.)
static int split_waves_to_a_unit(int head_dim) {
    static int known[8] = {0, 0, 0, 0, 0, 0, 0, 0};      // by head_dim / 32 - 1
    static std::mutex mutex;
    if (head_dim % 32 || head_dim < 32 || head_dim > 256) return 8;
    std::lock_guard<std::mutex> lock(mutex);
    int& n = known[head_dim / 32 - 1];
    if (n == 0) {
        int blocks = 0;
        hipError_t e = hipErrorInvalidValue;
        switch (head_dim) {
#define ASK(HD) case HD: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, attn_split16_kernel<HD>, 64, SPLIT16_LDS_BYTES); break;
            ASK(32) ASK(64) ASK(96) ASK(128) ASK(192) ASK(256)
#undef ASK
            default: break;
        }
        if (e != hipSuccess) (void)hipGetLastError();
        n = (e == hipSuccess && blocks >= 1) ? std::min(blocks, 32) : 8;
    }
    return n;
}

// Keys per wave of the split, by what the host knows: the number of single-token entries, the bound on their
// length, and (when it says so) how many keys they see together.  Measured on the 8B head shape (8 to 256 requests
// of 520 to 8000 keys, every chunk from 64 to 1024 keys) and on the 1B one: a compute unit holds so many of these
// waves at once (eight) and works through them in turns of that many.  Waves of one
// turn, all of the same length, end together, and the longest chunks that still fill half a turn are the fastest
// (a wave begins with a chain of trips to memory: lengths, page numbers, then keys); one wave more than a turn
// costs a second turn.  So: the smallest chunk that gives a unit no more than three quarters of a turn (the next
// length then still gives it more than a third); and when even chunks of 1024
// keys give more than a turn, 512 if the last turn would be far from full (many short waves share out evenly as they come).
// Against the best chunk of each case (also at sizes and lengths between those it was made from, at 4 and 8 heads
// to a kv head, 2 and 8 kv heads) this rule is within the 3 % that two timings of one case differ by, 6 % at worst;
// the rule before the first of this kind (128 keys, doubled while the waves kept all units busy, by the bound alone)
// lost 7.5 % on average and 19 % at worst.  The chunks of a request are never
// more than a quarter of what the merge takes.
// The number of keys moves with every step while a recorded graph holds the chunk it was recorded with: callers that
// record put this function's result into what they key their recordings by.  The scratch is sized by the smallest
// chunk the entries and the bound allow, taken at an eighth of the bound for every entry; fewer keys than that get
// that chunk too.
// LLMRS_SPLIT_CHUNK in the environment (64 to 1024, a power of two) takes the choice away from the rule, for measuring it.
extern "C" int llmrs_attention_split_chunk(long singles, int n_kv_heads, int head_dim, int max_seq_len, long single_keys) {
    if (const char* e = getenv("LLMRS_SPLIT_CHUNK")) {
        int c = atoi(e);
        if (c >= ATTN_CHUNK / 2 && c <= 8 * ATTN_CHUNK && (c & (c - 1)) == 0) return c;
    }
    double cus = (double)llmrs_compute_units();
    if (singles < 1) singles = 1;
    if (max_seq_len < 1) max_seq_len = 1;
    const double turn = split_waves_to_a_unit(head_dim);
    const int longest = 8 * ATTN_CHUNK;
    auto pick = [&](double keys) {
        // waves to a compute unit with chunks of c keys, every entry taken at the mean length; the last chunk of a
        // request counts as a wave unless it is so short that it is gone before it matters
        auto to_a_unit = [&](int c) {
            double q = keys / singles / c, whole = floor(q), rest = q - whole;
            return singles * n_kv_heads * (whole + (rest > 0.125 ? 1.0 : 0.0)) / cus;
        };
        const double full = turn * 1.001;
        // With the 16-column kernel a unit does best on about half a turn of waves, one to a SIMD: a full turn of
        // chunks half as long takes 2-7 % longer, a quarter of a turn of chunks twice as long 15-25 % (8 to 128
        // requests of 520 to 8000 keys, every chunk forced).  So chunks are doubled while a unit would get more than
        // three quarters of a turn: the next length still leaves it more than a third.
        const double enough = 0.75 * turn;
        int c = ATTN_CHUNK / 2;
        while (c < longest && to_a_unit(c) > enough) c *= 2;
        if (c == longest && to_a_unit(c) > full) {
            double last = fmod(to_a_unit(c), turn) / turn;
            if (last > 0.006 && last < 0.69) c /= 2;
        }
        while (c < longest && (max_seq_len + c - 1) / c > MERGE_MAX_CHUNKS / 4) c *= 2;
        return c;
    };
    double bound_keys = (double)singles * max_seq_len;
    int least = pick(bound_keys / 8.0);
    double keys = single_keys > 0 ? fmin((double)single_keys, bound_keys) : 0.75 * bound_keys;
    return std::max(pick(keys), least);
}

template <int HD>
static int launch(hipStream_t stream, const bf16* q, bf16* out, const bf16* kc, const bf16* vc, const int* table,
                  const int* positions, const int* q_starts, const int* seq_lens, int n_entries, float* scratch,
                  size_t scratch_bytes, int max_seq_len, int n_single, long single_keys, const AttnArgs& a) {
    int G = a.n_heads / a.n_kv_heads;
    int tpt = 32 / G;
    int chunk = llmrs_attention_split_chunk(n_single > 0 ? n_single : n_entries, a.n_kv_heads, HD, max_seq_len, single_keys);
    int max_chunks = max_seq_len > 0 ? (max_seq_len + chunk - 1) / chunk : 0;
    size_t need = (size_t)n_entries * a.n_heads * max_chunks * (HD + 2) * sizeof(float);
    // Split the single-token entries when the caller gave room for their partial results.
    int split = max_chunks > 0 && scratch != nullptr && seq_lens != nullptr && scratch_bytes >= need && max_chunks <= MERGE_MAX_CHUNKS && n_single != 0;
    // every entry brings one token, on the caller's word (n_single == n_entries): no tile work.  It is not read off
    // n_tokens == n_entries, which entries of two tokens and of none would satisfy as well.
    int only_single = split && n_single == n_entries && a.n_tokens == n_entries;
    // both kinds of work: the single tokens' kernels on the second stream, beside the tiles
    hipStream_t single_stream = stream;
    SideStream* side = nullptr;
    if (split && !only_single) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone) side = side_stream();
        else (void)hipGetLastError();
        if (side != nullptr) {
            if (hipEventRecord(side->fork, stream) == hipSuccess && hipStreamWaitEvent(side->stream, side->fork, 0) == hipSuccess)
                single_stream = side->stream;
            else { (void)hipGetLastError(); side = nullptr; }
        }
    }
    if (!only_single) {
        if constexpr (HD == 64 || HD == 128 || HD == 256) {
            // Over long caches blocks of eight waves, one to a unit: every tile of keys and values comes in for
            // twice the columns (a portion of 2048 tokens of the 8B shape over 32,768 / 65,536 / 131,072 keys:
            // 856 -> 893, 877 -> 934, 883 -> 947 TFLOP/s; over 8,192 keys 4 % slower, over 2,048 a quarter: the
            // blocks' lengths then differ too much for one block to a unit).
            bool wide = false;
            if constexpr (HD == 128) wide = max_seq_len >= ATTN_WIDE_FROM_KEYS;     // (head size 256 has no registers for two waves a SIMD)
            if (wide) {
                if constexpr (HD == 128) {
                    int btiles = a.n_tokens / (8 * tpt) + n_entries;
                    attn_tiles_lds_kernel<HD, 8><<<btiles * a.n_kv_heads, 512, 0, stream>>>(q, out, kc, vc, table, positions, q_starts,
                                                                                        n_entries, a, G, tpt, split, 0);
                }
            } else {
                int btiles = a.n_tokens / (4 * tpt) + n_entries;
                attn_tiles_lds_kernel<HD><<<btiles * a.n_kv_heads, 256, 0, stream>>>(q, out, kc, vc, table, positions, q_starts,
                                                                                     n_entries, a, G, tpt, split, llmrs_compute_units());
            }
        } else {
            int tiles = a.n_tokens / tpt + n_entries;
            int blocks = ((tiles + 3) / 4) * a.n_kv_heads;
            attn_tiles_kernel<HD><<<blocks, 256, 0, stream>>>(q, out, kc, vc, table, positions, q_starts, n_entries, a, G, tpt, split);
        }
    }
    if (split) {
        dim3 grid(n_entries, a.n_kv_heads, max_chunks);
        int plain = only_single && a.window == 0;
        if (G <= 16)
            attn_split16_kernel<HD><<<grid, 64, SPLIT16_LDS_BYTES, single_stream>>>(q, scratch, kc, vc, table, seq_lens, q_starts, a, G, max_chunks, chunk, plain);
        else
            attn_split_kernel<HD><<<grid, 64, 0, single_stream>>>(q, scratch, kc, vc, table, seq_lens, q_starts, a, G, max_chunks, chunk, plain);
        if (max_chunks > MERGE_ONE_WALK_CHUNKS && HD <= MERGE_GROUP_THREADS) {
            int threads = (HD / 2) * ((max_chunks + 3) / 4);          // groups of HD / 2 threads, a group for every four chunks
            threads = std::min(MERGE_GROUP_THREADS, std::max(HD, (threads + 63) / 64 * 64));
            attn_merge_groups_kernel<<<dim3(n_entries, a.n_heads), threads, 0, single_stream>>>(scratch, out, seq_lens, q_starts, a, max_chunks, chunk, plain);
        }
        else
            attn_merge_kernel<<<dim3(n_entries, a.n_heads), 64 * ((HD + 63) / 64), 0, single_stream>>>(scratch, out, seq_lens, q_starts, a, max_chunks, chunk, plain);
    }
    if (side != nullptr && single_stream != stream) {
        // the caller's stream goes on only when the second stream's kernels are done (they write other rows of `out`)
        if (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(stream, side->join, 0) != hipSuccess) {
            llmrs_fail("attention (mfma): cannot join the second stream: %s", hipGetErrorString(hipGetLastError()));
            (void)hipStreamSynchronize(side->stream);
            return -1;
        }
    }
    return 1;
}

int llmrs_attention_bf16_mfma(hipStream_t stream, const bf16* q, bf16* out, const bf16* k_cache, const bf16* v_cache,
                              const int* block_table, const int* token_entry, const int* positions,
                              const int* q_starts, const int* seq_lens, int n_entries, float* scratch,
                              size_t scratch_bytes, int max_seq_len, int n_single, long single_keys, const AttnArgs& a) {
    (void)token_entry;
    int G = a.n_heads / a.n_kv_heads;
    if (a.page_size != 16 || a.head_dim % 32 || G > 32 || q_starts == nullptr) return 0;
    if (a.q_stride % 8 || a.out_stride % 4 || ((uintptr_t)q & 15) || ((uintptr_t)out & 7)) return 0;
    if (n_entries > 65535 || a.n_kv_heads > 65535) return 0;
    int rc;
    switch (a.head_dim) {
#define CASE(HD) case HD: rc = launch<HD>(stream, q, out, k_cache, v_cache, block_table, positions, q_starts, seq_lens, n_entries, scratch, scratch_bytes, max_seq_len, n_single, single_keys, a); break;
        CASE(32) CASE(64) CASE(96) CASE(128) CASE(192) CASE(256)
#undef CASE
        default: return 0;
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        llmrs_fail("attention (mfma): launch failed: %s", hipGetErrorString(err));
        return -1;
    }
    return rc;
}
