// Writes the flat batch of one step into the pinned host buffer.
//
// A step holds, for each request in it, a contiguous run of its next tokens: whole prompts,
// portions of prompts and single decoded tokens side by side (crates/core/src/runner.rs:745-876):
//
//   input_ids    [T]     the tokens
//   positions    [T]     absolute position of each token
//   slot_mapping [T]     per cache group: page * page_size + position % page_size
//   cu_seqlens   [B+1]   prefix sums of the tokens per request
//   seq_lens     [B]     request length after this step (start + n)
//   block_table  [B, MB] per cache group, -1 where no page is held
//   state_slots  [B]     the request's fixed-size state slot
//   logits_rows  [R]     rows of the flat batch whose logits are wanted: every entry's `want`, then every entry's `more`
//   feedback_src [T]     -1, or: the token's id is the feedback_src-th token the last step sampled (still on the device)
//
// Padding (pad_to > B): a step of single rows that replays a captured graph of pad_to requests
// is filled up with requests of one token at position 0 that write no cache slot (slot -1) and
// read page 0, which always exists (crates/layers/src/exec.rs:388-426). Their state slot is max_reqs,
// one past the slots requests can hold: per-request state is allocated with that spare slot at its end.
// pad_batch() does the same for any step after it was filled: requests and tokens up to given counts (the made-up
// requests bring one token each, the last of them the rest), logits rows up to a given count.
#pragma once
#include <cstdint>
#include <cstring>
#include <string>

#include "cache_manager.hpp"

namespace dinfer {

constexpr int MAX_GROUPS = 8;

// Addresses inside the pinned buffer and the capacities they were sized for.
struct BatchBuffers {
    int32_t n_groups, max_tokens, max_reqs, max_rows;
    int32_t* input_ids;
    int32_t* positions;
    int32_t* cu_seqlens;
    int32_t* seq_lens;
    int32_t* state_slots;
    int32_t* logits_rows;
    int32_t* feedback_src;
    int64_t* slot_mapping[MAX_GROUPS];
    int32_t* block_table[MAX_GROUPS];
    int32_t max_blocks[MAX_GROUPS];
};

// What the host needs to know about the step it just described.
struct BatchFacts {
    int32_t num_tokens, num_reqs, num_rows, max_q_len, max_seq_len, num_singles;
};

// One request's share of a step. `tokens` has `count` ids; `want` has `n_want` indices into them.
struct EntryView {
    int64_t rid;
    int32_t start, count;
    const int32_t* tokens;
    const int32_t* want;
    int32_t n_want;
    int32_t feedback_src = -1;  // >= 0: the entry's last token is not known on the host yet; it is this one of the
                                // tokens the last step samples (its id in `tokens` is a placeholder)
    const int32_t* more = nullptr;  // n_more further wanted places, whose rows come after the `want` rows of
    int32_t n_more = 0;             // all entries
};

inline void fill_batch(const CacheManager& cache, const BatchBuffers& buf, const EntryView* entries, int n_entries,
                       int pad_to, BatchFacts* facts) {
    if (buf.n_groups != cache.num_groups() || buf.n_groups > MAX_GROUPS)
        throw Error(ERR_VALUE, "the batch buffers were laid out for another number of cache groups");
    int64_t T = 0, R = 0;
    for (int b = 0; b < n_entries; ++b) {
        if (entries[b].count <= 0) throw Error(ERR_VALUE, "entry " + std::to_string(b) + " brings no token to this step");
        T += entries[b].count;
        R += entries[b].n_want + entries[b].n_more;
    }
    const int B = n_entries;
    if (B == 0) throw Error(ERR_VALUE, "a step needs at least one request with at least one token");
    if (B > buf.max_reqs)
        throw Error(ERR_VALUE, std::to_string(B) + " requests in one step, the engine was built for " + std::to_string(buf.max_reqs));
    if (T > buf.max_tokens)
        throw Error(ERR_VALUE, std::to_string(T) + " tokens in one step, the engine was built for " + std::to_string(buf.max_tokens));
    if (R > buf.max_rows)
        throw Error(ERR_VALUE, "logits wanted at " + std::to_string(R) + " places, the engine was built for " + std::to_string(buf.max_rows));

    int t = 0, r = 0, max_q = 0, max_len = 0, singles = 0;
    buf.cu_seqlens[0] = 0;
    for (int b = 0; b < B; ++b) {
        const EntryView& e = entries[b];
        const int n = e.count;
        std::memcpy(buf.input_ids + t, e.tokens, sizeof(int32_t) * n);
        for (int i = 0; i < n; ++i) {
            buf.positions[t + i] = e.start + i;
            buf.feedback_src[t + i] = -1;
        }
        if (e.feedback_src >= 0) {
            buf.input_ids[t + n - 1] = 0;
            buf.feedback_src[t + n - 1] = e.feedback_src;
        }
        for (int g = 0; g < buf.n_groups; ++g) {
            const std::vector<int32_t>& tab = cache.block_table(e.rid, g);
            const int mb = buf.max_blocks[g];
            if (static_cast<int>(tab.size()) > mb)
                throw Error(ERR_VALUE, "entry " + std::to_string(b) + " holds " + std::to_string(tab.size()) +
                                           " pages, the block table has " + std::to_string(mb) + " columns");
            int32_t* row = buf.block_table[g] + static_cast<int64_t>(b) * mb;
            std::memcpy(row, tab.data(), sizeof(int32_t) * tab.size());
            for (int i = static_cast<int>(tab.size()); i < mb; ++i) row[i] = -1;
            cache.slot_mapping(e.rid, g, e.start, n, buf.slot_mapping[g] + t);
        }
        buf.cu_seqlens[b + 1] = t + n;
        buf.seq_lens[b] = e.start + n;
        buf.state_slots[b] = cache.slot_of(e.rid);
        for (int i = 0; i < e.n_want; ++i) {
            int w = e.want[i];
            if (w < 0 || w >= n)
                throw Error(ERR_VALUE, "entry " + std::to_string(b) + ": wanted place " + std::to_string(w) +
                                           " is outside its " + std::to_string(n) + " tokens");
            buf.logits_rows[r++] = t + w;
        }
        max_q = n > max_q ? n : max_q;
        max_len = e.start + n > max_len ? e.start + n : max_len;
        singles += n == 1;
        t += n;
    }
    for (int b = 0; b < B; ++b) {
        const EntryView& e = entries[b];
        for (int i = 0; i < e.n_more; ++i) {
            const int w = e.more[i];
            if (w < 0 || w >= e.count)
                throw Error(ERR_VALUE, "entry " + std::to_string(b) + ": wanted place " + std::to_string(w) +
                                           " is outside its " + std::to_string(e.count) + " tokens");
            buf.logits_rows[r++] = buf.cu_seqlens[b] + w;
        }
    }
    int Bp = B;
    if (pad_to > B) {
        const int P = pad_to;
        if (T != B || R != B || P > buf.max_reqs || P > buf.max_tokens || P > buf.max_rows)
            throw Error(ERR_VALUE, "only a step of single rows that all want logits can be padded");
        for (int b = B; b < P; ++b) {
            buf.input_ids[b] = 0;
            buf.feedback_src[b] = -1;
            buf.positions[b] = 0;
            buf.cu_seqlens[b + 1] = b + 1;
            buf.seq_lens[b] = 1;
            buf.state_slots[b] = buf.max_reqs;  // the spare slot: no request ever holds it
            buf.logits_rows[b] = b;
            for (int g = 0; g < buf.n_groups; ++g) {
                int32_t* row = buf.block_table[g] + static_cast<int64_t>(b) * buf.max_blocks[g];
                std::memset(row, 0, sizeof(int32_t) * buf.max_blocks[g]);
                buf.slot_mapping[g][b] = -1;
            }
        }
        singles += P - B;
        if (max_len < 1) max_len = 1;
        T = R = Bp = P;
    }
    facts->num_tokens = static_cast<int32_t>(T);
    facts->num_reqs = Bp;
    facts->num_rows = static_cast<int32_t>(R);
    facts->max_q_len = max_q;
    facts->max_seq_len = max_len;
    facts->num_singles = singles;
}

// Fills a step that fill_batch has written up to reqs requests, tokens tokens and rows logits rows, so that it
// can replay a graph captured for those counts. The made-up requests start at position 0, write no cache slot
// (slot -1), hold page 0 in every column of their block table (it always exists; what they read there counts for
// nothing) and the spare state slot; each brings one token, the last one whatever is still missing. The made-up
// logits rows point at the first made-up token (or at row 0). facts: the step's, brought up to date.
inline void pad_batch(const BatchBuffers& buf, BatchFacts* facts, int reqs, int tokens, int rows) {
    const int B = facts->num_reqs, T = facts->num_tokens, R = facts->num_rows;
    if (reqs < B || tokens < T || rows < R || reqs > buf.max_reqs || tokens > buf.max_tokens || rows > buf.max_rows)
        throw Error(ERR_VALUE, "a step can be padded up to the engine's sizes only, never cut");
    const int more_reqs = reqs - B, more_tokens = tokens - T;
    if ((more_reqs == 0) != (more_tokens == 0) || more_tokens < more_reqs)
        throw Error(ERR_VALUE, "made-up requests bring at least one token each, and made-up tokens need a request");
    int t = T, max_q = facts->max_q_len, max_len = facts->max_seq_len, singles = facts->num_singles;
    for (int b = B; b < reqs; ++b) {
        const int n = b + 1 < reqs ? 1 : tokens - t;
        for (int i = 0; i < n; ++i) {
            buf.input_ids[t + i] = 0;
            buf.feedback_src[t + i] = -1;
            buf.positions[t + i] = i;
            for (int g = 0; g < buf.n_groups; ++g) buf.slot_mapping[g][t + i] = -1;
        }
        for (int g = 0; g < buf.n_groups; ++g)
            std::memset(buf.block_table[g] + static_cast<int64_t>(b) * buf.max_blocks[g], 0,
                        sizeof(int32_t) * buf.max_blocks[g]);
        buf.cu_seqlens[b + 1] = t + n;
        buf.seq_lens[b] = n;
        buf.state_slots[b] = buf.max_reqs;
        max_q = n > max_q ? n : max_q;
        max_len = n > max_len ? n : max_len;
        singles += n == 1;
        t += n;
    }
    for (int r = R; r < rows; ++r) buf.logits_rows[r] = more_tokens > 0 ? T : 0;
    facts->num_tokens = tokens;
    facts->num_reqs = reqs;
    facts->num_rows = rows;
    facts->max_q_len = max_q;
    facts->max_seq_len = max_len;
    facts->num_singles = singles;
}

}  // namespace dinfer
