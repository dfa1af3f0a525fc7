// One step's batch, flattened into a single block of 32-bit words that goes to
// the device in one copy.
//
// A step holds R entries; entry r brings count[r] consecutive tokens of request
// slot[r], starting at position start[r].  The flat arrays are those of the
// reference's Batch (src/batch.rs:5-16) as build_batch fills them
// (src/serve/engine.rs:96-154), plus the request index of each token, the
// request's slot and, for each cache group, a slot map and a block table of its own.
#pragma once
#include <cstdint>
#include <vector>

#include "cache_manager.h"

namespace llmrs {

// Offsets, in words from the start of the block, of each array.
struct BatchLayout {
    int32_t header;       // [4]: T, R, n_want, 0
    int32_t tokens;       // [T]
    int32_t positions;    // [T]
    int32_t token_entry;  // [T]   index of the entry a token belongs to
    int32_t q_starts;     // [R+1] first token of each entry
    int32_t seq_lens;     // [R]   start + count: keys visible to the entry's last token
    int32_t slots;        // [R]   the request's stable slot
    int32_t want_rows;    // [n_want] rows of the T tokens whose logits are wanted
    int32_t sampling;     // [n_want*4] per wanted row: uniform, temperature (float bits), top_k, top_p (float bits)
    int32_t group0;       // per group: slot_map [T], then block_table [R * width]
    int32_t words;        // total
};

struct BatchEntry {
    int slot;
    int start;
    int count;
};

// Words needed for a batch of the given sizes; `widths[g]` is the block table's
// row length in group g.
BatchLayout batch_layout(int T, int R, int n_want, const std::vector<int>& widths);
int group_slot_map_offset(const BatchLayout& l, int g, int T, int R, const std::vector<int>& widths);
int group_table_offset(const BatchLayout& l, int g, int T, int R, const std::vector<int>& widths);

// Row length each group's block table needs for these entries (at least 1).
std::vector<int> table_widths(const CacheManager& cache, const std::vector<BatchEntry>& entries);

// Fills `words` (layout.words long).  `tokens` has the entries' tokens in order,
// `want_rows` indexes into them.  Pages must have been ensured before.
void fill_batch(const CacheManager& cache, const std::vector<BatchEntry>& entries,
                const int32_t* tokens, const int32_t* want_rows, int n_want,
                const std::vector<int>& widths, const BatchLayout& layout, int32_t* words);

}  // namespace llmrs
