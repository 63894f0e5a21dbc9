// The cache manager: pages per group of layers, a block table per request and group, and a
// slot of fixed size per request.
//
// Groups. Layers whose caches have the same page geometry and the same need ("all keys" or
// "the last W keys") form a group. A group has its own pool of pages and each request has one
// block table per group; a page id is valid in every layer of its group
// (models/qwen3/src/model.rs:604-612, crates/core/src/kv/manager.rs:52-56).
//
// Allocation (crates/core/src/kv/manager.rs:203-281): before a step a request asks for the
// pages its next tokens need; the answer is all-or-nothing over all groups. A decode token
// that stays inside its last page allocates nothing.
//
// Giving back. All pages and the slot when the request ends or is preempted
// (sched/mod.rs:783-803,672-680). In a window group also, after each step, every page whose
// keys all lie before the window of the request's next token; its block-table entry becomes
// -1 and is never read again.
//
// Prefix cache (optional; crates/core/src/kv/hash.rs:20-60, kv/manager.rs:150-199,288-335). A full page
// of a request's tokens gets a name: a hash of the tokens in it chained to the name of the page
// before it, so a name stands for the whole prefix up to and including that page. commit() names
// the pages a step has filled; lookup() gives a new request the longest run of named pages that
// matches the start of its prompt (never all of it: the last token is always computed), so those
// tokens need not be computed again. A named page that nobody holds waits at the tail of the
// free list and is handed out last. Names are checked against the stored tokens and the
// parent's name, so two prefixes whose hashes collide are still told apart. Only for groups
// that keep every key (a window group gives pages back while the request lives).
//
// State slots (in the manner of crates/layers/src/exec.rs:253-333). Each live request holds
// one index in [0, max_seqs) for its whole life. A slot handed out is reported by
// take_fresh_slots() so that the engine zero-fills its state before the first step that uses it.
#pragma once
#include <algorithm>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "block_pool.hpp"

namespace dinfer {

struct GroupSpec {
    int page_size;
    int num_blocks;
    int window;  // < 0: every key of the request is kept; W >= 1: the last W keys
};

class CacheManager {
public:
    CacheManager(std::vector<GroupSpec> groups, int max_seqs, bool prefix_cache = false)
        : groups_(std::move(groups)), max_seqs_(max_seqs), prefix_cache_(prefix_cache) {
        if (max_seqs <= 0) throw Error(ERR_VALUE, "max_seqs must be positive");
        for (const GroupSpec& g : groups_) {
            if (g.page_size <= 0) throw Error(ERR_VALUE, "a page holds at least one token");
            pools_.emplace_back(g.num_blocks);
        }
        for (int s = max_seqs - 1; s >= 0; --s) free_slots_.push_back(s);
        if (prefix_cache_) {
            if (groups_.empty()) throw Error(ERR_VALUE, "a prefix cache needs a cache group");
            for (const GroupSpec& g : groups_) {
                if (g.window >= 0) throw Error(ERR_VALUE, "the prefix cache needs groups that keep every key");
                if (g.page_size != groups_[0].page_size)
                    throw Error(ERR_VALUE, "the prefix cache needs one page size in all groups");
                named_tokens_.emplace_back(static_cast<size_t>(g.num_blocks) * g.page_size, 0);
                named_parent_.emplace_back(g.num_blocks, 0);
                named_check_.emplace_back(g.num_blocks, 0);
            }
        }
    }

    bool prefix_cache() const { return prefix_cache_; }

    int num_groups() const { return static_cast<int>(groups_.size()); }
    int max_seqs() const { return max_seqs_; }
    const GroupSpec& group(int g) const { return groups_.at(g); }
    const BlockPool& pool(int g) const { return pools_.at(g); }
    int num_live() const { return static_cast<int>(reqs_.size()); }

    // ---- requests
    bool has(int64_t rid) const { return reqs_.count(rid) != 0; }
    bool can_admit() const { return !free_slots_.empty(); }

    int admit(int64_t rid) {
        if (has(rid)) throw Error(ERR_KEY, "the request is already live");
        if (free_slots_.empty())
            throw Error(ERR_RUNTIME, "all " + std::to_string(max_seqs_) + " request slots are taken");
        int slot = free_slots_.back();
        free_slots_.pop_back();
        fresh_slots_.push_back(slot);
        Req r;
        r.tables.resize(groups_.size());
        r.slot = slot;
        reqs_.emplace(rid, std::move(r));
        return slot;
    }

    std::vector<int> take_fresh_slots() {
        std::vector<int> out;
        out.swap(fresh_slots_);
        return out;
    }

    int slot_of(int64_t rid) const { return find(rid).slot; }

    std::vector<int64_t> live_requests() const {
        std::vector<int64_t> out;
        for (const auto& kv : reqs_) out.push_back(kv.first);
        return out;
    }

    // ---- pages
    // Per group, how many new pages the tokens [num_computed, num_computed + num_new) need.
    void pages_needed(int64_t rid, int64_t num_computed, int64_t num_new, int* need) const {
        const Req& r = find(rid);
        int64_t end = num_computed + num_new;
        for (size_t g = 0; g < groups_.size(); ++g) {
            int64_t want = (end + groups_[g].page_size - 1) / groups_[g].page_size;
            need[g] = static_cast<int>(std::max<int64_t>(0, want - static_cast<int64_t>(r.tables[g].size())));
        }
    }

    // Pages for tokens [num_computed, num_computed + num_new) in every group, or nothing at all.
    bool allocate(int64_t rid, int64_t num_computed, int64_t num_new) {
        if (num_new <= 0) throw Error(ERR_VALUE, "a step feeds at least one token per request");
        Req& r = find(rid);
        need_.resize(groups_.size());
        pages_needed(rid, num_computed, num_new, need_.data());
        for (size_t g = 0; g < groups_.size(); ++g)
            if (need_[g] > pools_[g].num_free()) return false;
        for (size_t g = 0; g < groups_.size(); ++g) pools_[g].allocate(need_[g], r.tables[g]);
        r.num_tokens = std::max(r.num_tokens, num_computed + num_new);
        return true;
    }

    // After a step: frees the pages of window groups that the token at position num_computed and
    // all later ones cannot see. Returns how many were freed.
    int release_passed(int64_t rid, int64_t num_computed) {
        Req& r = find(rid);
        int freed = 0;
        for (size_t g = 0; g < groups_.size(); ++g) {
            const GroupSpec& gs = groups_[g];
            if (gs.window < 0) continue;
            std::vector<int32_t>& tab = r.tables[g];
            int64_t first_key = std::max<int64_t>(0, num_computed - gs.window + 1);
            size_t first = std::min<size_t>(static_cast<size_t>(first_key / gs.page_size), tab.size());
            scratch_.clear();
            for (size_t i = 0; i < first; ++i)
                if (tab[i] >= 0) scratch_.push_back(tab[i]);
            if (scratch_.empty()) continue;
            pools_[g].free(scratch_.data(), static_cast<int>(scratch_.size()));
            freed += static_cast<int>(scratch_.size());
            for (size_t i = 0; i < first; ++i) tab[i] = -1;
        }
        return freed;
    }

    // Gives back everything the request holds, the last page first, so the tail of a request is
    // what the next allocation takes (kv/manager.rs:338-345).
    void free(int64_t rid) {
        auto it = reqs_.find(rid);
        if (it == reqs_.end()) throw Error(ERR_KEY, "the request is not live");
        Req& r = it->second;
        for (size_t g = 0; g < groups_.size(); ++g) {
            scratch_.clear();
            for (auto p = r.tables[g].rbegin(); p != r.tables[g].rend(); ++p)
                if (*p >= 0) scratch_.push_back(*p);
            pools_[g].free(scratch_.data(), static_cast<int>(scratch_.size()));
        }
        free_slots_.push_back(r.slot);
        fresh_slots_.erase(std::remove(fresh_slots_.begin(), fresh_slots_.end(), r.slot), fresh_slots_.end());
        reqs_.erase(it);
    }

    // ---- prefix cache
    // For a request that holds no page yet: takes the longest run of named pages matching the start of
    // tokens[0, n), at most (n - 1) / page_size of them, and returns how many tokens they cover.
    int64_t lookup(int64_t rid, const int32_t* tokens, int64_t n) {
        Req& r = find(rid);
        if (!prefix_cache_) return 0;
        for (const auto& t : r.tables)
            if (!t.empty()) throw Error(ERR_RUNTIME, "a prefix is looked up before the request holds pages");
        const int ps = groups_[0].page_size;
        const int64_t most = n > 0 ? (n - 1) / ps : 0;
        uint64_t name = 0, chk = 0;
        int64_t got = 0;
        std::vector<int32_t> hit(groups_.size());
        for (; got < most; ++got) {
            uint64_t nn, nc;
            name_page(name, chk, tokens + got * ps, ps, &nn, &nc);
            bool all = true;
            for (size_t g = 0; g < groups_.size() && all; ++g) {
                const int b = pools_[g].find(nn);
                all = b >= 0 && named_check_[g][b] == nc && named_parent_[g][b] == name &&
                      std::equal(tokens + got * ps, tokens + (got + 1) * ps, named_tokens_[g].begin() + static_cast<size_t>(b) * ps);
                hit[g] = b;
            }
            if (!all) break;
            for (size_t g = 0; g < groups_.size(); ++g) {
                pools_[g].touch(hit[g]);
                r.tables[g].push_back(hit[g]);
            }
            name = nn;
            chk = nc;
        }
        r.num_named = got;
        r.last_name = name;
        r.last_check = chk;
        r.num_tokens = got * ps;
        return got * ps;
    }

    // After a step: the pages that tokens[0, num_computed) fill completely get their names.
    void commit(int64_t rid, const int32_t* tokens, int64_t num_computed) {
        if (!prefix_cache_) return;
        Req& r = find(rid);
        const int ps = groups_[0].page_size;
        const int64_t full = num_computed / ps;
        for (; r.num_named < full; ++r.num_named) {
            const int64_t i = r.num_named;
            uint64_t nn, nc;
            name_page(r.last_name, r.last_check, tokens + i * ps, ps, &nn, &nc);
            for (size_t g = 0; g < groups_.size(); ++g) {
                const int b = r.tables[g].at(i);
                // if another page carries the name already, this one stays nameless (its content is a duplicate)
                if (!pools_[g].has_name(b) && pools_[g].set_name(b, nn)) {
                    named_check_[g][b] = nc;
                    named_parent_[g][b] = r.last_name;
                    std::copy(tokens + i * ps, tokens + (i + 1) * ps, named_tokens_[g].begin() + static_cast<size_t>(b) * ps);
                }
            }
            r.last_name = nn;
            r.last_check = nc;
        }
    }

    // ---- views for the step
    const std::vector<int32_t>& block_table(int64_t rid, int g) const { return find(rid).tables.at(g); }

    // Cache slots (page * page_size + offset) of positions start .. start + n - 1.
    void slot_mapping(int64_t rid, int g, int64_t start, int64_t n, int64_t* out) const {
        const std::vector<int32_t>& tab = find(rid).tables.at(g);
        const int64_t ps = groups_[g].page_size;
        for (int64_t i = 0; i < n; ++i) {
            int64_t pos = start + i;
            int64_t page = pos / ps;
            if (pos < 0 || page >= static_cast<int64_t>(tab.size()))
                throw Error(ERR_RUNTIME, "position " + std::to_string(pos) + " has no page allocated");
            int32_t b = tab[page];
            if (b < 0)
                throw Error(ERR_RUNTIME, "position " + std::to_string(pos) + " lies in a page that was given back");
            out[i] = b * ps + pos % ps;
        }
    }

    // Invariants: no page lost, none held twice, every held page in exactly one table; the same for slots.
    void check() const {
        for (size_t g = 0; g < groups_.size(); ++g) {
            const BlockPool& pool = pools_[g];
            pool.check();
            // a page is in as many block tables as it has references (more than one only for shared prefixes)
            std::vector<int32_t> uses(pool.num_blocks(), 0);
            for (const auto& kv : reqs_) {
                for (int32_t b : kv.second.tables[g]) {
                    if (b < 0) continue;
                    std::string where = "group " + std::to_string(g) + ": page " + std::to_string(b);
                    if (b >= pool.num_blocks()) throw Error(ERR_ASSERT, where + " does not exist");
                    if (!pool.is_held(b)) throw Error(ERR_ASSERT, where + " of a live request is on the free list");
                    if (++uses[b] > 1 && !prefix_cache_) throw Error(ERR_ASSERT, where + " is in two block tables");
                }
            }
            int held = 0;
            for (int b = 0; b < pool.num_blocks(); ++b) {
                if (uses[b] != pool.ref_count(b))
                    throw Error(ERR_ASSERT, "group " + std::to_string(g) + ": page " + std::to_string(b) + " is in " +
                                                std::to_string(uses[b]) + " block tables and has " +
                                                std::to_string(pool.ref_count(b)) + " references");
                held += uses[b] > 0;
            }
            if (held + pool.num_free() != pool.num_blocks())
                throw Error(ERR_ASSERT, "group " + std::to_string(g) + ": " +
                                            std::to_string(pool.num_blocks() - pool.num_free() - held) + " pages are lost");
        }
        std::vector<uint8_t> slot_seen(max_seqs_, 0);
        size_t n = 0;
        auto mark = [&](int s) {
            if (s < 0 || s >= max_seqs_ || slot_seen[s]) throw Error(ERR_ASSERT, "a state slot is held twice");
            slot_seen[s] = 1;
            ++n;
        };
        for (const auto& kv : reqs_) mark(kv.second.slot);
        for (int s : free_slots_) mark(s);
        if (n != static_cast<size_t>(max_seqs_)) throw Error(ERR_ASSERT, "a state slot is lost");
    }

private:
    struct Req {
        std::vector<std::vector<int32_t>> tables;
        int64_t num_tokens = 0;  // tokens for which pages have been allocated
        int slot = -1;
        int64_t num_named = 0;   // leading pages that carry a name (or were tried)
        uint64_t last_name = 0, last_check = 0;  // of page num_named - 1
    };

    const Req& find(int64_t rid) const {
        auto it = reqs_.find(rid);
        if (it == reqs_.end()) throw Error(ERR_KEY, "the request is not live");
        return it->second;
    }
    Req& find(int64_t rid) { return const_cast<Req&>(static_cast<const CacheManager*>(this)->find(rid)); }

    std::vector<GroupSpec> groups_;
    std::vector<BlockPool> pools_;
    int max_seqs_;
    std::vector<int> free_slots_, fresh_slots_;
    std::unordered_map<int64_t, Req> reqs_;
    // Two independent 64-bit hashes of (the parent's two, the page's tokens): one is the name, the other
    // is kept beside the page and compared on a hit.
    static uint64_t mix(uint64_t x) {
        x += 0x9e3779b97f4a7c15ull;
        x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
        x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
        return x ^ (x >> 31);
    }
    static void name_page(uint64_t parent, uint64_t parent_check, const int32_t* tokens, int n, uint64_t* name,
                          uint64_t* check) {
        uint64_t a = mix(parent ^ 0x243f6a8885a308d3ull), b = mix(parent_check ^ 0x13198a2e03707344ull);
        for (int i = 0; i < n; ++i) {
            const uint64_t t = static_cast<uint32_t>(tokens[i]);
            a = mix(a ^ t);
            b = mix(b + (t << 1 | 1) * 0xa4093822299f31d0ull);
        }
        *name = a;
        *check = b;
    }

    bool prefix_cache_ = false;
    std::vector<std::vector<int32_t>> named_tokens_;   // per group: [page][page_size] tokens of named pages
    std::vector<std::vector<uint64_t>> named_parent_;  // per group: the name of the page before
    std::vector<std::vector<uint64_t>> named_check_;   // per group: the second hash
    std::vector<int> need_;
    std::vector<int32_t> scratch_;
};

}  // namespace dinfer
