// The C interface over the host core's classes; see dinfer_host.h for the contract.
#include "dinfer_host.h"

#include <cstring>
#include <string>
#include <vector>

#include "scheduler.hpp"

using namespace dinfer;

static_assert(DH_MAX_GROUPS == MAX_GROUPS, "group capacity of the C struct and of the core differ");
static_assert(sizeof(dh_batch_buffers) == sizeof(BatchBuffers), "dh_batch_buffers must mirror BatchBuffers");
static_assert(sizeof(dh_batch_facts) == sizeof(BatchFacts), "dh_batch_facts must mirror BatchFacts");
static_assert(sizeof(dh_sched_options) == sizeof(SchedOptions), "dh_sched_options must mirror SchedOptions");
static_assert(sizeof(dh_scheduled) == sizeof(Scheduled), "dh_scheduled must mirror Scheduled");
static_assert(sizeof(dh_update_result) == sizeof(UpdateResult), "dh_update_result must mirror UpdateResult");

namespace {

thread_local std::string g_error;

template <class F>
int32_t guarded(F&& f) {
    try {
        return f();
    } catch (const Error& e) {
        g_error = e.what();
        return -static_cast<int32_t>(e.kind);
    } catch (const std::out_of_range& e) {
        g_error = std::string("index out of range: ") + e.what();
        return -ERR_VALUE;
    } catch (const std::exception& e) {
        g_error = e.what();
        return -ERR_RUNTIME;
    }
}

template <class It>
int32_t copy_out(It first, It last, int32_t* out, int32_t capacity) {
    int32_t n = 0;
    for (; first != last; ++first, ++n)
        if (n < capacity) out[n] = static_cast<int32_t>(*first);
    return n;
}

struct SchedulerBox {
    Scheduler sched;
    std::vector<EntryView> entries;
    std::vector<int32_t> wants;
    std::vector<UpdateResult> results;
    SchedulerBox(const SchedOptions& o, CacheManager* c, const int32_t* eos, int n) : sched(o, c, eos, n) {}
};

BlockPool* P(void* p) { return static_cast<BlockPool*>(p); }
CacheManager* C(void* p) { return static_cast<CacheManager*>(p); }
SchedulerBox* S(void* p) { return static_cast<SchedulerBox*>(p); }

}  // namespace

extern "C" {

const char* dh_last_error(void) { return g_error.c_str(); }

// ---- pool
void* dh_pool_create(int32_t num_blocks) {
    void* out = nullptr;
    guarded([&] { out = new BlockPool(num_blocks); return 0; });
    return out;
}
void dh_pool_destroy(void* pool) { delete P(pool); }
int32_t dh_pool_num_free(void* pool) { return P(pool)->num_free(); }
int32_t dh_pool_allocate(void* pool, int32_t n, int32_t* out) {
    return guarded([&] {
        std::vector<int32_t> got;
        if (!P(pool)->allocate(n, got)) return 0;
        std::memcpy(out, got.data(), sizeof(int32_t) * got.size());
        return 1;
    });
}
int32_t dh_pool_free(void* pool, const int32_t* ids, int32_t n) {
    return guarded([&] { P(pool)->free(ids, n); return 0; });
}
int32_t dh_pool_free_list(void* pool, int32_t* out, int32_t capacity) {
    const auto& f = P(pool)->free_list();
    return copy_out(f.begin(), f.end(), out, capacity);
}
int32_t dh_pool_is_held(void* pool, int32_t page) { return P(pool)->is_held(page) ? 1 : 0; }
int32_t dh_pool_check(void* pool) {
    return guarded([&] { P(pool)->check(); return 0; });
}

// ---- cache manager
void* dh_cache_create(int32_t n_groups, const int32_t* page_sizes, const int32_t* num_blocks, const int32_t* windows,
                      int32_t max_seqs, int32_t prefix_cache) {
    void* out = nullptr;
    guarded([&] {
        std::vector<GroupSpec> groups;
        for (int g = 0; g < n_groups; ++g) groups.push_back({page_sizes[g], num_blocks[g], windows[g]});
        out = new CacheManager(std::move(groups), max_seqs, prefix_cache != 0);
        return 0;
    });
    return out;
}
void dh_cache_destroy(void* cache) { delete C(cache); }
int32_t dh_cache_has(void* cache, int64_t rid) { return C(cache)->has(rid) ? 1 : 0; }
int32_t dh_cache_can_admit(void* cache) { return C(cache)->can_admit() ? 1 : 0; }
int32_t dh_cache_admit(void* cache, int64_t rid) {
    return guarded([&] { return C(cache)->admit(rid); });
}
int32_t dh_cache_take_fresh_slots(void* cache, int32_t* out, int32_t capacity) {
    return guarded([&] {
        if (capacity < C(cache)->max_seqs()) throw Error(ERR_VALUE, "room for max_seqs slots is needed");
        std::vector<int> s = C(cache)->take_fresh_slots();
        return copy_out(s.begin(), s.end(), out, capacity);
    });
}
int32_t dh_cache_slot_of(void* cache, int64_t rid) {
    return guarded([&] { return C(cache)->slot_of(rid); });
}
int32_t dh_cache_live_requests(void* cache, int64_t* out, int32_t capacity) {
    std::vector<int64_t> ids = C(cache)->live_requests();
    for (size_t i = 0; i < ids.size() && static_cast<int32_t>(i) < capacity; ++i) out[i] = ids[i];
    return static_cast<int32_t>(ids.size());
}
int32_t dh_cache_pages_needed(void* cache, int64_t rid, int64_t num_computed, int64_t num_new, int32_t* need) {
    return guarded([&] { C(cache)->pages_needed(rid, num_computed, num_new, need); return 0; });
}
int32_t dh_cache_allocate(void* cache, int64_t rid, int64_t num_computed, int64_t num_new) {
    return guarded([&] { return C(cache)->allocate(rid, num_computed, num_new) ? 1 : 0; });
}
int32_t dh_cache_release_passed(void* cache, int64_t rid, int64_t num_computed) {
    return guarded([&] { return C(cache)->release_passed(rid, num_computed); });
}
int32_t dh_cache_free(void* cache, int64_t rid) {
    return guarded([&] { C(cache)->free(rid); return 0; });
}
int32_t dh_cache_block_table(void* cache, int64_t rid, int32_t group, int32_t* out, int32_t capacity) {
    return guarded([&] {
        const auto& t = C(cache)->block_table(rid, group);
        return copy_out(t.begin(), t.end(), out, capacity);
    });
}
int32_t dh_cache_slot_mapping(void* cache, int64_t rid, int32_t group, int64_t start, int64_t n, int64_t* out) {
    return guarded([&] {
        if (group < 0 || group >= C(cache)->num_groups()) throw Error(ERR_VALUE, "no such cache group");
        C(cache)->slot_mapping(rid, group, start, n, out);
        return 0;
    });
}
int32_t dh_cache_num_free(void* cache, int32_t group) {
    return guarded([&] { return C(cache)->pool(group).num_free(); });
}
int32_t dh_cache_free_list(void* cache, int32_t group, int32_t* out, int32_t capacity) {
    return guarded([&] {
        const auto& f = C(cache)->pool(group).free_list();
        return copy_out(f.begin(), f.end(), out, capacity);
    });
}
int32_t dh_cache_check(void* cache) {
    return guarded([&] { C(cache)->check(); return 0; });
}
int64_t dh_cache_lookup(void* cache, int64_t rid, const int32_t* tokens, int64_t n) {
    int64_t got = 0;
    const int32_t rc = guarded([&] { got = C(cache)->lookup(rid, tokens, n); return 0; });
    return rc < 0 ? rc : got;
}
int32_t dh_cache_commit(void* cache, int64_t rid, const int32_t* tokens, int64_t num_computed) {
    return guarded([&] { C(cache)->commit(rid, tokens, num_computed); return 0; });
}

// ---- batch
int32_t dh_batch_fill(void* cache, const dh_batch_buffers* buf, int32_t n, const int64_t* rids, const int32_t* starts,
                      const int32_t* counts, const int32_t* tokens, const int32_t* want_counts, const int32_t* wants,
                      int32_t pad_to, dh_batch_facts* facts) {
    return guarded([&] {
        std::vector<EntryView> entries;
        entries.reserve(n > 0 ? n : 0);
        int64_t t = 0, w = 0;
        for (int b = 0; b < n; ++b) {
            if (counts[b] < 0 || want_counts[b] < 0) throw Error(ERR_VALUE, "negative count in entry " + std::to_string(b));
            entries.push_back({rids[b], starts[b], counts[b], tokens + t, wants + w, want_counts[b]});
            t += counts[b];
            w += want_counts[b];
        }
        fill_batch(*C(cache), *reinterpret_cast<const BatchBuffers*>(buf), entries.data(), n, pad_to,
                   reinterpret_cast<BatchFacts*>(facts));
        return 0;
    });
}

int32_t dh_batch_pad(const dh_batch_buffers* buf, dh_batch_facts* facts, int32_t reqs, int32_t tokens, int32_t rows) {
    return guarded([&] {
        pad_batch(*reinterpret_cast<const BatchBuffers*>(buf), reinterpret_cast<BatchFacts*>(facts), reqs, tokens, rows);
        return 0;
    });
}

// ---- scheduler
void* dh_sched_create(const dh_sched_options* opt, void* cache, const int32_t* eos, int32_t n_eos) {
    void* out = nullptr;
    guarded([&] {
        SchedOptions o;
        std::memcpy(&o, opt, sizeof(o));
        out = new SchedulerBox(o, C(cache), eos, n_eos);
        return 0;
    });
    return out;
}
void dh_sched_destroy(void* sched) { delete S(sched); }

int32_t dh_sched_add(void* sched, int64_t rid, const int32_t* prompt, int32_t n_prompt, int32_t max_tokens,
                     int32_t min_tokens, int32_t ignore_eos, const int32_t* stop_ids, int32_t n_stop,
                     int32_t every_row) {
    return guarded([&] {
        auto r = std::make_unique<Request>();
        r->id = rid;
        r->tokens.assign(prompt, prompt + (n_prompt > 0 ? n_prompt : 0));
        r->max_tokens = max_tokens;
        r->min_tokens = min_tokens;
        r->ignore_eos = ignore_eos != 0;
        r->stop_ids.assign(stop_ids, stop_ids + (n_stop > 0 ? n_stop : 0));
        r->every_row = every_row != 0;
        S(sched)->sched.add(std::move(r));
        return 0;
    });
}
int32_t dh_sched_abort(void* sched, int64_t rid) {
    return guarded([&] { S(sched)->sched.abort(rid); return 0; });
}
int32_t dh_sched_forget(void* sched, int64_t rid) {
    return guarded([&] { S(sched)->sched.forget(rid); return 0; });
}
int32_t dh_sched_has_unfinished(void* sched) { return S(sched)->sched.has_unfinished() ? 1 : 0; }
int32_t dh_sched_request_info(void* sched, int64_t rid, dh_request_info* out) {
    return guarded([&] {
        const Request* r = S(sched)->sched.get(rid);
        if (!r) throw Error(ERR_KEY, "the scheduler does not know the request");
        *out = {r->num_prompt, r->num_tokens(), r->num_computed, r->status, r->reason, r->preemptions, r->num_cached};
        return 0;
    });
}
int32_t dh_sched_queue(void* sched, int32_t running, int64_t* out, int32_t capacity) {
    int32_t n = 0;
    auto put = [&](const Request* r) {
        if (n < capacity) out[n] = r->id;
        ++n;
    };
    if (running)
        for (const Request* r : S(sched)->sched.running()) put(r);
    else
        for (const Request* r : S(sched)->sched.waiting()) put(r);
    return n;
}
int32_t dh_sched_schedule(void* sched, int32_t* n_out) {
    return guarded([&] {
        const StepPlan& p = S(sched)->sched.schedule();
        n_out[0] = static_cast<int32_t>(p.scheduled.size());
        n_out[1] = static_cast<int32_t>(p.preempted.size());
        n_out[2] = static_cast<int32_t>(p.force_finished.size());
        return 0;
    });
}
int32_t dh_sched_can_look_ahead(void* sched) {
    return guarded([&] { return S(sched)->sched.can_look_ahead() ? 1 : 0; });
}
int32_t dh_sched_schedule_ahead(void* sched, int32_t* n_out) {
    return guarded([&] {
        const StepPlan& p = S(sched)->sched.schedule_ahead();
        n_out[0] = static_cast<int32_t>(p.scheduled.size());
        n_out[1] = static_cast<int32_t>(p.preempted.size());
        n_out[2] = static_cast<int32_t>(p.force_finished.size());
        return 0;
    });
}
int32_t dh_sched_plan(void* sched, dh_scheduled* scheduled, int64_t* preempted, int64_t* finished_ids,
                      int32_t* finished_reasons) {
    const StepPlan& p = S(sched)->sched.plan();
    if (!p.scheduled.empty()) std::memcpy(scheduled, p.scheduled.data(), sizeof(Scheduled) * p.scheduled.size());
    for (size_t i = 0; i < p.preempted.size(); ++i) preempted[i] = p.preempted[i];
    for (size_t i = 0; i < p.force_finished.size(); ++i) {
        finished_ids[i] = p.force_finished[i].first;
        finished_reasons[i] = p.force_finished[i].second;
    }
    return 0;
}
int32_t dh_sched_fill(void* sched, const dh_batch_buffers* buf, int32_t pad_to, dh_batch_facts* facts) {
    return guarded([&] {
        SchedulerBox* s = S(sched);
        s->sched.plan_entries(s->entries, s->wants);
        fill_batch(*s->sched.cache(), *reinterpret_cast<const BatchBuffers*>(buf), s->entries.data(),
                   static_cast<int>(s->entries.size()), pad_to, reinterpret_cast<BatchFacts*>(facts));
        return 0;
    });
}
int32_t dh_sched_update(void* sched, const int32_t* sampled, int32_t n_sampled, dh_update_result* out, int32_t capacity) {
    return guarded([&] {
        SchedulerBox* s = S(sched);
        s->results.clear();
        s->sched.update(sampled, n_sampled, s->results);
        int32_t n = static_cast<int32_t>(s->results.size());
        if (n > capacity) throw Error(ERR_VALUE, "room for one result per scheduled request is needed");
        if (n) std::memcpy(out, s->results.data(), sizeof(UpdateResult) * n);
        return n;
    });
}

}  // extern "C"
