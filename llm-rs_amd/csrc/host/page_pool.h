// A pool of page ids with a LIFO free list.  The list starts as n-1..0 so that
// pops yield 0,1,2,... and a page given back is the next one handed out, as in
// the reference (src/kv_pool.rs:43, :51-61).  Unlike the reference it knows which
// ids are out, and refuses a page that is given back twice or was never its own.
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace llmrs {

class PagePool {
public:
    explicit PagePool(int num_pages) : held_(num_pages, 0) {
        free_.reserve(num_pages);
        for (int i = num_pages - 1; i >= 0; --i) free_.push_back(i);
    }
    int total() const { return (int)held_.size(); }
    int available() const { return (int)free_.size(); }
    bool is_held(int page) const { return page >= 0 && page < total() && held_[page]; }

    int take() {
        if (free_.empty()) return -1;
        int page = free_.back();
        free_.pop_back();
        held_[page] = 1;
        return page;
    }
    void give_back(int page) {
        if (page < 0 || page >= total())
            throw std::logic_error("page " + std::to_string(page) + " is not of this pool");
        if (!held_[page])
            throw std::logic_error("page " + std::to_string(page) + " given back twice");
        held_[page] = 0;
        free_.push_back(page);
    }

private:
    std::vector<int32_t> free_;
    std::vector<uint8_t> held_;
};

}  // namespace llmrs
