#include "cache_manager.h"

#include <stdexcept>

namespace llmrs {

CacheManager::CacheManager(const std::vector<GroupSpec>& groups, int max_requests)
    : groups_(groups), in_use_(max_requests, 0), tables_(max_requests) {
    if (max_requests <= 0) throw std::invalid_argument("max_requests must be positive");
    for (const auto& g : groups_) {
        if (g.page_size <= 0) throw std::invalid_argument("page_size must be positive");
        if (g.num_pages <= 0) throw std::invalid_argument("num_pages must be positive");
        if (g.window < 0) throw std::invalid_argument("window must not be negative");
        pools_.emplace_back(g.num_pages);
    }
    for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);
    for (auto& t : tables_) t.resize(groups_.size());
}

void CacheManager::check_slot(int slot) const {
    if (!slot_in_use(slot)) throw std::logic_error("slot " + std::to_string(slot) + " is not in use");
}

int CacheManager::acquire_slot() {
    if (free_slots_.empty()) return -1;
    int slot = free_slots_.back();
    free_slots_.pop_back();
    in_use_[slot] = 1;
    ++slots_used_;
    return slot;
}

void CacheManager::release_pages(int slot) {
    check_slot(slot);
    for (int g = 0; g < num_groups(); ++g) {
        for (int32_t page : tables_[slot][g])
            if (page >= 0) pools_[g].give_back(page);
        tables_[slot][g].clear();
    }
}

void CacheManager::release_slot(int slot) {
    release_pages(slot);
    in_use_[slot] = 0;
    --slots_used_;
    free_slots_.push_back(slot);
}

int CacheManager::pages_held(int slot, int g) const {
    check_slot(slot);
    int n = 0;
    for (int32_t page : tables_[slot][g]) n += page >= 0;
    return n;
}

void CacheManager::drop_passed(int slot, int g, int start) {
    int ps = groups_[g].page_size;
    int keep_from = first_visible(g, start) / ps;  // first logical page still visible
    auto& t = tables_[slot][g];
    for (int i = 0; i < keep_from && i < (int)t.size(); ++i) {
        if (t[i] >= 0) {
            pools_[g].give_back(t[i]);
            t[i] = -1;
        }
    }
}

int CacheManager::pages_needed(int g, int start, int count) const {
    int ps = groups_[g].page_size;
    int first = first_visible(g, start) / ps;
    int last = (start + count + ps - 1) / ps;
    return last - first;
}

bool CacheManager::ensure(int slot, int start, int count) {
    check_slot(slot);
    if (start < 0 || count < 0) throw std::invalid_argument("negative position or count");
    // Pages that no query of this or any later step can see go back first; that
    // never fails and may be what lets this request (or another) go on.
    for (int g = 0; g < num_groups(); ++g) drop_passed(slot, g, start);
    for (int g = 0; g < num_groups(); ++g) {
        int ps = groups_[g].page_size;
        int need = (start + count + ps - 1) / ps - (int)tables_[slot][g].size();
        // Logical pages below the visible range are never taken, so a request that
        // starts late in a window group (after a recompute) holds holes there.
        int first = first_visible(g, start) / ps;
        int have = (int)tables_[slot][g].size();
        int fresh = 0;
        for (int i = have; i < have + (need > 0 ? need : 0); ++i) fresh += i >= first;
        if (fresh > pools_[g].available()) return false;
    }
    for (int g = 0; g < num_groups(); ++g) {
        int ps = groups_[g].page_size;
        int last = (start + count + ps - 1) / ps;
        int first = first_visible(g, start) / ps;
        auto& t = tables_[slot][g];
        while ((int)t.size() < last) t.push_back((int)t.size() >= first ? pools_[g].take() : -1);
    }
    return true;
}

}  // namespace llmrs
