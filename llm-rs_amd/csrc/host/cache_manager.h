// Pages and block tables for every live request, and the stable slot a request
// keeps for its life.
//
// Layers whose caches have the same needs form a group.  Each group has a page
// pool and, for each request, a block table of its own: entry i is the page that
// holds positions [i*page_size, (i+1)*page_size), or -1 once a window has passed
// it and the page went back to the pool.  A group with window w keeps only the
// pages that a query at the request's next position can still see (keys at
// positions > p - w); a group with window 0 keeps all.
//
// Reference: PagedKVPool + ensure_blocks (src/kv_pool.rs:12-95) is the single
// group, all-keys case; RequestTable (src/serve/engine.rs:69-92) is the stable
// slot.  Groups, windows and the ownership checks have no counterpart there.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "page_pool.h"

namespace llmrs {

struct GroupSpec {
    int page_size;
    int num_pages;
    int window;  // 0: every key stays visible
};

class CacheManager {
public:
    CacheManager(const std::vector<GroupSpec>& groups, int max_requests);

    int num_groups() const { return (int)groups_.size(); }
    const GroupSpec& group(int g) const { return groups_[g]; }
    int max_requests() const { return (int)in_use_.size(); }
    int pages_free(int g) const { return pools_[g].available(); }
    int pages_total(int g) const { return pools_[g].total(); }

    // A slot for a new request, or -1 when all are taken.
    int acquire_slot();
    // Gives the request's pages and its slot back.
    void release_slot(int slot);
    bool slot_in_use(int slot) const { return slot >= 0 && slot < max_requests() && in_use_[slot]; }
    int slots_in_use() const { return slots_used_; }

    // Pages for positions [start, start+count) in every group, after giving back
    // what a window has passed for a query at `start`.  All or nothing: when any
    // group lacks pages nothing new is taken (src/kv_pool.rs:83-95).
    bool ensure(int slot, int start, int count);
    // Gives back every page of the request; it keeps its slot (recompute later).
    void release_pages(int slot);
    // Pages a request would have to hold at once to run [start, start+count).
    int pages_needed(int g, int start, int count) const;

    const std::vector<int32_t>& table(int slot, int g) const { return tables_[slot][g]; }
    int pages_held(int slot, int g) const;
    // First position whose page group g still has to hold for a query at `pos`.
    int first_visible(int g, int pos) const {
        int w = groups_[g].window;
        return (w <= 0 || pos + 1 <= w) ? 0 : pos + 1 - w;
    }

private:
    void check_slot(int slot) const;
    void drop_passed(int slot, int g, int start);

    std::vector<GroupSpec> groups_;
    std::vector<PagePool> pools_;
    std::vector<uint8_t> in_use_;
    std::vector<int32_t> free_slots_;
    int slots_used_ = 0;
    std::vector<std::vector<std::vector<int32_t>>> tables_;  // [slot][group][logical page]
};

}  // namespace llmrs
