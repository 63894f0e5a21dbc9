/* C interface of the host core (page pools, cache manager, scheduler, batch fill).
 *
 * Every function that can fail returns a negative number on failure: minus the kind of the
 * error (1 unknown or duplicate request, 2 the state does not allow the call, 3 an argument
 * is out of range, 4 an invariant is broken). dh_last_error() then gives the text, valid
 * until the same thread's next failing call. Requests are named by 64-bit numbers that the
 * caller chooses. Objects are not thread-safe: one thread at a time per object. */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* dh_last_error(void);

/* ---- a pool of pages on its own */
void* dh_pool_create(int32_t num_blocks);
void dh_pool_destroy(void* pool);
int32_t dh_pool_num_free(void* pool);
int32_t dh_pool_allocate(void* pool, int32_t n, int32_t* out);            /* 1 done, 0 not enough pages */
int32_t dh_pool_free(void* pool, const int32_t* ids, int32_t n);
int32_t dh_pool_free_list(void* pool, int32_t* out, int32_t capacity);   /* returns the count */
int32_t dh_pool_is_held(void* pool, int32_t page);
int32_t dh_pool_check(void* pool);

/* ---- cache manager. windows[g] < 0: the group keeps every key. prefix_cache: pages are named after the
 * tokens they hold, so that a later request with the same start need not compute them again */
void* dh_cache_create(int32_t n_groups, const int32_t* page_sizes, const int32_t* num_blocks, const int32_t* windows,
                      int32_t max_seqs, int32_t prefix_cache);
void dh_cache_destroy(void* cache);
int32_t dh_cache_has(void* cache, int64_t rid);
int32_t dh_cache_can_admit(void* cache);
int32_t dh_cache_admit(void* cache, int64_t rid);                         /* the state slot */
int32_t dh_cache_take_fresh_slots(void* cache, int32_t* out, int32_t capacity);
int32_t dh_cache_slot_of(void* cache, int64_t rid);
int32_t dh_cache_live_requests(void* cache, int64_t* out, int32_t capacity);
int32_t dh_cache_pages_needed(void* cache, int64_t rid, int64_t num_computed, int64_t num_new, int32_t* need);
int32_t dh_cache_allocate(void* cache, int64_t rid, int64_t num_computed, int64_t num_new); /* 1 done, 0 no pages */
int32_t dh_cache_release_passed(void* cache, int64_t rid, int64_t num_computed);            /* pages freed */
int32_t dh_cache_free(void* cache, int64_t rid);
int32_t dh_cache_block_table(void* cache, int64_t rid, int32_t group, int32_t* out, int32_t capacity); /* length */
int32_t dh_cache_slot_mapping(void* cache, int64_t rid, int32_t group, int64_t start, int64_t n, int64_t* out);
int32_t dh_cache_num_free(void* cache, int32_t group);
int32_t dh_cache_free_list(void* cache, int32_t group, int32_t* out, int32_t capacity);
int32_t dh_cache_check(void* cache);
/* prefix cache: tokens of the request from its first; lookup returns how many of them are covered by cached pages
 * (the request must be admitted and hold no page yet); commit names the pages that tokens[0, num_computed) fill */
int64_t dh_cache_lookup(void* cache, int64_t rid, const int32_t* tokens, int64_t n);
int32_t dh_cache_commit(void* cache, int64_t rid, const int32_t* tokens, int64_t num_computed);

/* ---- the flat batch of a step, written into the caller's pinned buffer */
#define DH_MAX_GROUPS 8
typedef struct {
    int32_t n_groups, max_tokens, max_reqs, max_rows;
    int32_t* input_ids;
    int32_t* positions;
    int32_t* cu_seqlens;
    int32_t* seq_lens;
    int32_t* state_slots;
    int32_t* logits_rows;
    int32_t* feedback_src; /* per token: -1, or which of the last step's sampled tokens (on the device) it is */
    int64_t* slot_mapping[DH_MAX_GROUPS];
    int32_t* block_table[DH_MAX_GROUPS];
    int32_t max_blocks[DH_MAX_GROUPS];
} dh_batch_buffers;

typedef struct {
    int32_t num_tokens, num_reqs, num_rows, max_q_len, max_seq_len, num_singles;
} dh_batch_facts;

/* entries b = 0 .. n-1: request rids[b] feeds counts[b] tokens from position starts[b]; their
 * ids follow each other in `tokens`, the wanted places (indices into the entry's tokens) in `wants`. */
int32_t dh_batch_fill(void* cache, const dh_batch_buffers* buf, int32_t n, const int64_t* rids, const int32_t* starts,
                      const int32_t* counts, const int32_t* tokens, const int32_t* want_counts, const int32_t* wants,
                      int32_t pad_to, dh_batch_facts* facts);

/* Fills a written step up to `reqs` requests, `tokens` tokens and `rows` logits rows with made-up requests that
 * write nothing (one token each, the last one the rest), so that it can replay a graph captured for those counts. */
int32_t dh_batch_pad(const dh_batch_buffers* buf, dh_batch_facts* facts, int32_t reqs, int32_t tokens, int32_t rows);

/* ---- scheduler */
typedef struct {
    int32_t max_num_batched_tokens, max_num_seqs, max_model_len, prefill_tokens_per_step,
        long_prefill_token_threshold, enable_chunked_prefill, decode_exempt_from_budget, enable_prefix_caching,
        prefill_chunk_alignment, max_logits_rows;
} dh_sched_options;

/* rows_from, num_rows: prompt positions at which logits are wanted as well; their rows follow the sampling rows */
typedef struct { int64_t id; int32_t start, num_new, samples, rows_from, num_rows; } dh_scheduled;
typedef struct { int64_t id; int32_t token, reason; } dh_update_result;
/* status: 0 waiting, 1 running, 2 preempted, 3 finished. reason: 0 none, 1 stop, 2 length, 3 abort */
typedef struct { int32_t num_prompt, num_tokens, num_computed, status, reason, preemptions, num_cached; } dh_request_info;

void* dh_sched_create(const dh_sched_options* opt, void* cache, const int32_t* eos, int32_t n_eos);
void dh_sched_destroy(void* sched);
/* every_row: logits are wanted at every prompt position whose next token is in the prompt (needs max_logits_rows >
 * max_num_seqs) */
int32_t dh_sched_add(void* sched, int64_t rid, const int32_t* prompt, int32_t n_prompt, int32_t max_tokens,
                     int32_t min_tokens, int32_t ignore_eos, const int32_t* stop_ids, int32_t n_stop,
                     int32_t every_row);
int32_t dh_sched_abort(void* sched, int64_t rid);
int32_t dh_sched_forget(void* sched, int64_t rid);
int32_t dh_sched_has_unfinished(void* sched);
int32_t dh_sched_request_info(void* sched, int64_t rid, dh_request_info* out);
int32_t dh_sched_queue(void* sched, int32_t running, int64_t* out, int32_t capacity);  /* ids in queue order */
/* plans a step; counts of the three lists go to n_out[3]; read them with dh_sched_plan */
int32_t dh_sched_schedule(void* sched, int32_t* n_out);
/* 1 if the next step can be planned while the last planned step still runs (before its dh_sched_update) */
int32_t dh_sched_can_look_ahead(void* sched);
/* plans that next step: every request of the running step that goes on decodes once more, its input token being
 * the one the running step samples (a placeholder on the host; the batch names its place among those tokens).
 * The next dh_sched_update is the running step's, the one after it this step's. */
int32_t dh_sched_schedule_ahead(void* sched, int32_t* n_out);
int32_t dh_sched_plan(void* sched, dh_scheduled* scheduled, int64_t* preempted, int64_t* finished_ids,
                      int32_t* finished_reasons);
/* writes the planned step into the batch buffers straight from the requests' tokens */
int32_t dh_sched_fill(void* sched, const dh_batch_buffers* buf, int32_t pad_to, dh_batch_facts* facts);
/* sampled: one token per sampling request of the plan, in order. Returns the number of results. */
int32_t dh_sched_update(void* sched, const int32_t* sampled, int32_t n_sampled, dh_update_result* out, int32_t capacity);

#ifdef __cplusplus
}
#endif
