// A pool of cache pages.
//
// allocate(n) is all-or-nothing and takes pages from the head of the free list; free(ids)
// puts the pages back at the head in the order given, so pages that were just given back
// are the next ones handed out (crates/core/src/kv/block_pool.rs:128-147,160-182; this
// engine has no prefix cache, so there is no LRU tail). A page is held by at most one
// owner; freeing a page that is not held is an error and changes nothing.
#pragma once
#include <cstdint>
#include <deque>
#include <string>
#include <vector>

#include "errors.hpp"

namespace dinfer {

class BlockPool {
public:
    explicit BlockPool(int num_blocks) : held_(check_size(num_blocks), 0) {
        for (int b = 0; b < num_blocks; ++b) free_.push_back(b);
    }

    int num_blocks() const { return static_cast<int>(held_.size()); }
    int num_free() const { return static_cast<int>(free_.size()); }
    bool is_held(int b) const { return b >= 0 && b < num_blocks() && held_[b]; }
    const std::deque<int32_t>& free_list() const { return free_; }

    // Appends n page ids to `out` and returns true, or returns false and changes nothing.
    bool allocate(int n, std::vector<int32_t>& out) {
        if (n < 0) throw Error(ERR_VALUE, "cannot allocate a negative number of pages");
        if (n > num_free()) return false;
        for (int i = 0; i < n; ++i) {
            int32_t b = free_.front();
            free_.pop_front();
            held_[b] = 1;
            out.push_back(b);
        }
        return true;
    }

    void free(const int32_t* ids, int n) {
        for (int i = 0; i < n; ++i) {
            int32_t b = ids[i];
            if (!is_held(b)) {
                for (int j = 0; j < i; ++j) held_[ids[j]] = 1;  // undo: a failed call changes nothing
                throw Error(ERR_RUNTIME, "page " + std::to_string(b) + " is freed but not held");
            }
            held_[b] = 0;
        }
        for (int i = n - 1; i >= 0; --i) free_.push_front(ids[i]);
    }

    // Every page is either free exactly once or held (never both, never neither).
    void check() const {
        std::vector<uint8_t> on_list(held_.size(), 0);
        for (int32_t b : free_) {
            if (b < 0 || b >= num_blocks()) throw Error(ERR_ASSERT, "the free list holds page " + std::to_string(b));
            if (on_list[b]) throw Error(ERR_ASSERT, "a page is on the free list twice");
            on_list[b] = 1;
        }
        for (int b = 0; b < num_blocks(); ++b) {
            if (static_cast<bool>(held_[b]) == static_cast<bool>(on_list[b]))
                throw Error(ERR_ASSERT, "page " + std::to_string(b) + (held_[b] ? " is held and free" : " is lost"));
        }
    }

private:
    static int check_size(int n) {
        if (n <= 0) throw Error(ERR_VALUE, "a pool needs at least one page, got " + std::to_string(n));
        return n;
    }
    std::deque<int32_t> free_;
    std::vector<uint8_t> held_;
};

}  // namespace dinfer
