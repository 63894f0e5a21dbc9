// A pool of cache pages.
//
// allocate(n) is all-or-nothing and takes pages from the head of the free list; free(ids)
// gives up one reference to each page, and a page nobody refers to any more goes back on the
// free list: at the head, in the order given, if its content has no name (so pages that were
// just given back are the next ones handed out), at the tail if it has (so named content is
// evicted last, oldest first) (crates/core/src/kv/block_pool.rs:128-147,160-182).
//
// Named content (the prefix cache): set_name(page, name) records that the page holds the keys
// and values of a block of tokens known by a 64-bit name; find(name) gives the page back as
// long as it has not been handed out again; touch(page) takes a reference to it, reviving it
// from the free list if nobody held it (block_pool.rs:150-157). allocate() forgets the name
// of a page it hands out.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "errors.hpp"

namespace dinfer {

class BlockPool {
public:
    explicit BlockPool(int num_blocks)
        : ref_(check_size(num_blocks), 0), prev_(num_blocks), next_(num_blocks), named_(num_blocks, 0), name_(num_blocks, 0) {
        for (int b = 0; b < num_blocks; ++b) {
            prev_[b] = b - 1;
            next_[b] = b + 1 < num_blocks ? b + 1 : -1;
        }
        head_ = 0;
        tail_ = num_blocks - 1;
        num_free_ = num_blocks;
    }

    int num_blocks() const { return static_cast<int>(ref_.size()); }
    int num_free() const { return num_free_; }
    bool is_held(int b) const { return b >= 0 && b < num_blocks() && ref_[b] > 0; }
    int ref_count(int b) const { return ref_.at(b); }

    std::vector<int32_t> free_list() const {
        std::vector<int32_t> out;
        for (int b = head_; b >= 0; b = next_[b]) out.push_back(b);
        return out;
    }

    // Appends n page ids to `out` and returns true, or returns false and changes nothing.
    bool allocate(int n, std::vector<int32_t>& out) {
        if (n < 0) throw Error(ERR_VALUE, "cannot allocate a negative number of pages");
        if (n > num_free_) return false;
        for (int i = 0; i < n; ++i) {
            const int b = head_;
            unlink(b);
            forget_name(b);
            ref_[b] = 1;
            out.push_back(b);
        }
        return true;
    }

    void free(const int32_t* ids, int n) {
        for (int i = 0; i < n; ++i) {
            const int32_t b = ids[i];
            if (!is_held(b)) {
                for (int j = 0; j < i; ++j) ++ref_[ids[j]];  // undo: a failed call changes nothing
                throw Error(ERR_RUNTIME, "page " + std::to_string(b) + " is freed but not held");
            }
            --ref_[b];
        }
        // unnamed pages to the head in the order given (so walk backwards), named ones to the tail
        for (int i = n - 1; i >= 0; --i)
            if (ref_[ids[i]] == 0 && !named_[ids[i]] && !on_list(ids[i])) push_front(ids[i]);
        for (int i = 0; i < n; ++i)
            if (ref_[ids[i]] == 0 && named_[ids[i]] && !on_list(ids[i])) push_back(ids[i]);
    }

    // ---- named content
    bool has_name(int b) const { return named_.at(b) != 0; }
    uint64_t name_of(int b) const { return name_.at(b); }

    int find(uint64_t name) const {
        auto it = by_name_.find(name);
        return it == by_name_.end() ? -1 : it->second;
    }

    // The page must be held. Returns false (and changes nothing) if another page has the name already.
    bool set_name(int b, uint64_t name) {
        if (!is_held(b)) throw Error(ERR_RUNTIME, "only a held page can be named");
        if (named_[b]) return name_[b] == name;
        if (!by_name_.emplace(name, b).second) return false;
        named_[b] = 1;
        name_[b] = name;
        return true;
    }

    // One more reference to a page; a page on the free list comes off it.
    void touch(int b) {
        if (b < 0 || b >= num_blocks()) throw Error(ERR_VALUE, "no such page");
        if (ref_[b] == 0) unlink(b);
        ++ref_[b];
    }

    // Every page is either on the free list exactly once or held (never both, never neither);
    // names point at pages that carry them.
    void check() const {
        std::vector<uint8_t> seen(ref_.size(), 0);
        int count = 0, last = -1;
        for (int b = head_; b >= 0; b = next_[b]) {
            if (b >= num_blocks()) throw Error(ERR_ASSERT, "the free list holds page " + std::to_string(b));
            if (seen[b]) throw Error(ERR_ASSERT, "a page is on the free list twice");
            if (prev_[b] != last) throw Error(ERR_ASSERT, "the free list is broken at page " + std::to_string(b));
            seen[b] = 1;
            last = b;
            if (++count > num_blocks()) break;
        }
        if (last != tail_ || count != num_free_) throw Error(ERR_ASSERT, "the free list and its count disagree");
        for (int b = 0; b < num_blocks(); ++b) {
            if (ref_[b] < 0) throw Error(ERR_ASSERT, "page " + std::to_string(b) + " has a negative count");
            if ((ref_[b] > 0) == static_cast<bool>(seen[b]))
                throw Error(ERR_ASSERT, "page " + std::to_string(b) + (ref_[b] > 0 ? " is held and free" : " is lost"));
        }
        size_t named = 0;
        for (int b = 0; b < num_blocks(); ++b) {
            if (!named_[b]) continue;
            ++named;
            auto it = by_name_.find(name_[b]);
            if (it == by_name_.end() || it->second != b) throw Error(ERR_ASSERT, "a page's name is not in the index");
        }
        if (named != by_name_.size()) throw Error(ERR_ASSERT, "the name index holds a page that has no name");
    }

private:
    static int check_size(int n) {
        if (n <= 0) throw Error(ERR_VALUE, "a pool needs at least one page, got " + std::to_string(n));
        return n;
    }
    bool on_list(int b) const { return prev_[b] != -2; }
    void unlink(int b) {
        const int p = prev_[b], n = next_[b];
        if (p >= 0) next_[p] = n; else head_ = n;
        if (n >= 0) prev_[n] = p; else tail_ = p;
        prev_[b] = next_[b] = -2;  // off the list
        --num_free_;
    }
    void push_front(int b) {
        prev_[b] = -1;
        next_[b] = head_;
        if (head_ >= 0) prev_[head_] = b; else tail_ = b;
        head_ = b;
        ++num_free_;
    }
    void push_back(int b) {
        next_[b] = -1;
        prev_[b] = tail_;
        if (tail_ >= 0) next_[tail_] = b; else head_ = b;
        tail_ = b;
        ++num_free_;
    }
    void forget_name(int b) {
        if (!named_[b]) return;
        by_name_.erase(name_[b]);
        named_[b] = 0;
    }

    std::vector<int32_t> ref_, prev_, next_;
    std::vector<uint8_t> named_;
    std::vector<uint64_t> name_;
    std::unordered_map<uint64_t, int32_t> by_name_;
    int head_ = -1, tail_ = -1, num_free_ = 0;
};

}  // namespace dinfer
