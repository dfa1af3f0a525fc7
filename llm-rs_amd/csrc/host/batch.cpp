#include "batch.h"

#include <algorithm>
#include <stdexcept>
#include <string>

namespace llmrs {

BatchLayout batch_layout(int T, int R, int n_want, const std::vector<int>& widths) {
    BatchLayout l{};
    int at = 0;
    auto take = [&](int n) { int o = at; at += n; return o; };
    l.header = take(4);
    l.tokens = take(T);
    l.positions = take(T);
    l.token_entry = take(T);
    l.q_starts = take(R + 1);
    l.seq_lens = take(R);
    l.slots = take(R);
    l.want_rows = take(n_want);
    l.sampling = take(n_want * 4);
    l.group0 = at;
    for (int w : widths) take(T + R * w);
    l.words = at;
    return l;
}

int group_slot_map_offset(const BatchLayout& l, int g, int T, int R, const std::vector<int>& widths) {
    int at = l.group0;
    for (int i = 0; i < g; ++i) at += T + R * widths[i];
    return at;
}

int group_table_offset(const BatchLayout& l, int g, int T, int R, const std::vector<int>& widths) {
    return group_slot_map_offset(l, g, T, R, widths) + T;
}

std::vector<int> table_widths(const CacheManager& cache, const std::vector<BatchEntry>& entries) {
    std::vector<int> widths(cache.num_groups(), 1);
    for (const auto& e : entries)
        for (int g = 0; g < cache.num_groups(); ++g)
            widths[g] = std::max(widths[g], (int)cache.table(e.slot, g).size());
    return widths;
}

void fill_batch(const CacheManager& cache, const std::vector<BatchEntry>& entries,
                const int32_t* tokens, const int32_t* want_rows, int n_want,
                const std::vector<int>& widths, const BatchLayout& l, int32_t* w) {
    int R = (int)entries.size();
    int T = 0;
    for (const auto& e : entries) T += e.count;
    std::fill(w, w + l.words, 0);
    w[l.header + 0] = T;
    w[l.header + 1] = R;
    w[l.header + 2] = n_want;
    int t = 0;
    for (int r = 0; r < R; ++r) {
        const auto& e = entries[r];
        if (e.count <= 0) throw std::invalid_argument("an entry brings no tokens");
        w[l.q_starts + r] = t;
        w[l.seq_lens + r] = e.start + e.count;
        w[l.slots + r] = e.slot;
        for (int i = 0; i < e.count; ++i, ++t) {
            w[l.tokens + t] = tokens[t];
            w[l.positions + t] = e.start + i;
            w[l.token_entry + t] = r;
        }
    }
    w[l.q_starts + R] = T;
    for (int i = 0; i < n_want; ++i) {
        if (want_rows[i] < 0 || want_rows[i] >= T) throw std::invalid_argument("wanted row outside the batch");
        w[l.want_rows + i] = want_rows[i];
    }
    for (int g = 0; g < cache.num_groups(); ++g) {
        int ps = cache.group(g).page_size;
        int32_t* slot_map = w + group_slot_map_offset(l, g, T, R, widths);
        int32_t* tables = w + group_table_offset(l, g, T, R, widths);
        int tt = 0;
        for (int r = 0; r < R; ++r) {
            const auto& e = entries[r];
            const auto& table = cache.table(e.slot, g);
            if ((int)table.size() > widths[g]) throw std::logic_error("block table wider than its row");
            for (int i = 0; i < e.count; ++i, ++tt) {
                int p = e.start + i;
                if (p / ps >= (int)table.size() || table[p / ps] < 0)
                    throw std::logic_error("position " + std::to_string(p) + " of slot " + std::to_string(e.slot) +
                                           " has no page in group " + std::to_string(g));
                slot_map[tt] = table[p / ps] * ps + p % ps;  // src/batch.rs:31-34
            }
            // Entries past the table and pages a window has passed read as page 0
            // (src/serve/engine.rs:131-137 pads with 0 too): no kernel looks at them,
            // and one that did by mistake would read valid memory and fail a test
            // rather than fault the device.
            for (int i = 0; i < widths[g]; ++i)
                tables[r * widths[g] + i] = (i < (int)table.size() && table[i] >= 0) ? table[i] : 0;
        }
    }
}

}  // namespace llmrs
