// Continuous batching: admits requests, cuts prompts into portions under a token budget,
// decodes, finishes and frees. It sees the cache only through the cache manager. The rules are
// the reference's (crates/core/src/sched/mod.rs):
//
//   * no separate prefill and decode phases: each step a request gets min(tokens it still has
//     to compute, what the budget allows) tokens (:1-11,377);
//   * running requests first, in admission order, then waiting ones first-come first-served
//     while budget, request slots and pages last (:350-477);
//   * a decode row (one token, with history) does not consume the budget when
//     decode_exempt_from_budget is set (:351,361-365);
//   * when pages run out for a running request, the last running request is preempted: its
//     pages are freed, it forgets what it computed and goes to the front of the waiting queue,
//     to recompute prompt and outputs later (:402-436,672-680). If the requester is itself the
//     last one it is skipped this step while others run, and finished with "length" if it is
//     alone (:414-432). A waiting request that cannot get pages waits (:571-573). A step that
//     preempted admits nobody (:473);
//   * finish: eos or stop id (after min_tokens, unless ignore_eos), max_tokens outputs, or
//     max_model_len tokens (:816-828).
#pragma once
#include <algorithm>
#include <cstdint>
#include <deque>
#include <memory>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "cache_manager.hpp"
#include "step_batch.hpp"

namespace dinfer {

struct SchedOptions {
    int32_t max_num_batched_tokens;
    int32_t max_num_seqs;
    int32_t max_model_len;
    int32_t prefill_tokens_per_step;       // 0: no cap
    int32_t long_prefill_token_threshold;  // 0: no cap
    int32_t enable_chunked_prefill;
    int32_t decode_exempt_from_budget;
    int32_t enable_prefix_caching;  // needs a cache manager built with a prefix cache
    int32_t prefill_chunk_alignment;  // a portion that does not end its request's tokens ends at a multiple of this (<= 1: anywhere)
    int32_t max_logits_rows;  // rows of logits a step can return (0: max_num_seqs); what exceeds max_num_seqs is free
                              // for the prompt positions of requests that want logits at each of them
};

enum Status : int32_t { WAITING = 0, RUNNING = 1, PREEMPTED = 2, FINISHED = 3 };
enum Reason : int32_t { NO_REASON = 0, STOP = 1, LENGTH = 2, ABORT = 3 };

struct Request {
    int64_t id = 0;
    std::vector<int32_t> tokens;  // prompt, then outputs
    int32_t num_prompt = 0;
    int32_t num_computed = 0;
    Status status = WAITING;
    Reason reason = NO_REASON;
    int32_t max_tokens = 0, min_tokens = 0;
    bool ignore_eos = false;
    std::vector<int32_t> stop_ids;
    int32_t preemptions = 0;
    int32_t num_cached = 0;  // tokens of the prompt found in the prefix cache at the last admission
    // Look-ahead: the step that samples this request's next token is still running and the step after it is planned
    // already. `tokens` then ends with a placeholder (-1) whose value that running step brings; pending_src is the
    // place of this request among the running step's sampled tokens. ending: the running step's token is the
    // request's last whatever it is (max_tokens or max_model_len), so no further step is planned for it.
    int32_t pending = 0, pending_src = -1;
    bool ending = false;
    // every_row: logits are wanted at every position of the prompt whose next token is in the prompt too (the
    // log-probabilities of a prompt, crates/core/src/sample.rs:103-105), beside the row that samples. Such a request
    // takes nothing from the prefix cache, and its portions are cut to the rows a step has to spare. rows_done:
    // positions below this have had theirs (a request that is preempted computes them again, silently).
    bool every_row = false;
    int32_t rows_done = 0;

    int32_t num_tokens() const { return static_cast<int32_t>(tokens.size()); }
    int32_t num_output() const { return num_tokens() - num_prompt; }
};

struct Scheduled {
    int64_t id;
    int32_t start;    // tokens computed before this step
    int32_t num_new;  // tokens this step feeds
    int32_t samples;  // the step reaches the end of the known tokens, so a token is sampled
    int32_t rows_from, num_rows;  // logits are wanted at the num_rows positions from rows_from on as well (after the
                                  // rows of all sampling requests, in the order of the plan)
};

// (feedback: for each scheduled request, the place among the sampled tokens of the step before whose value its last
// token is, or -1: known only where that step was still running when this one was planned)
struct StepPlan {
    std::vector<Scheduled> scheduled;  // running first, then newly admitted
    std::vector<int64_t> preempted;
    std::vector<std::pair<int64_t, Reason>> force_finished;  // ended by the scheduler itself
    std::vector<int32_t> feedback;
    bool open = false;  // planned and not yet updated
};

struct UpdateResult {
    int64_t id;
    int32_t token;   // -1: nothing sampled
    int32_t reason;  // Reason; NO_REASON while the request goes on
};

class Scheduler {
public:
    Scheduler(const SchedOptions& opt, CacheManager* cache, const int32_t* eos, int n_eos)
        : opt_(opt), cache_(cache), eos_(eos, eos + n_eos) {
        if (opt_.enable_prefix_caching && !cache_->prefix_cache())
            throw Error(ERR_VALUE, "prefix caching is asked for but the cache manager was built without it");
    }

    // ---- intake
    void add(std::unique_ptr<Request> req) {
        if (reqs_.count(req->id)) throw Error(ERR_KEY, "the request id is in use");
        if (req->tokens.empty()) throw Error(ERR_VALUE, "a prompt needs at least one token");
        req->num_prompt = req->num_tokens();
        if (req->num_prompt >= opt_.max_model_len)
            throw Error(ERR_VALUE, "prompt of " + std::to_string(req->num_prompt) +
                                       " tokens leaves no room for output within max_model_len " +
                                       std::to_string(opt_.max_model_len));
        if (req->every_row) {
            if (spare_rows() <= 0)
                throw Error(ERR_VALUE, "logits at every prompt position need rows beyond one per request: "
                                       "max_logits_rows must exceed max_num_seqs");
            if (!opt_.enable_chunked_prefill && req->num_prompt - 1 > spare_rows())
                throw Error(ERR_VALUE, "without chunked prefill a prompt of " + std::to_string(req->num_prompt) +
                                           " tokens needs " + std::to_string(req->num_prompt - 1) + " spare rows of logits");
        }
        req->status = WAITING;
        req->num_computed = 0;
        req->rows_done = 0;
        Request* r = req.get();
        reqs_.emplace(r->id, std::move(req));
        waiting_.push_back(r);
    }

    bool has_unfinished() const { return !waiting_.empty() || !running_.empty(); }
    const Request* get(int64_t id) const {
        auto it = reqs_.find(id);
        return it == reqs_.end() ? nullptr : it->second.get();
    }
    const std::deque<Request*>& waiting() const { return waiting_; }
    const std::vector<Request*>& running() const { return running_; }
    const StepPlan& plan() const { return plan_; }
    const CacheManager* cache() const { return cache_; }

    void abort(int64_t id) {
        auto it = reqs_.find(id);
        if (it != reqs_.end()) finish(it->second.get(), ABORT);
    }

    // A finished request stays readable until the owner has taken its final state.
    void forget(int64_t id) {
        auto it = reqs_.find(id);
        if (it != reqs_.end() && it->second->status == FINISHED) reqs_.erase(it);
    }

    // A portion that stops short of the request's last token is shortened so that it ends at a multiple of the
    // alignment (layers that work in chunks of their own want portions to end where their chunks end, in the manner
    // of crates/core/src/sched/mod.rs:146-166); 0 if not even one aligned position fits.
    int64_t aligned(int64_t computed, int64_t n, int64_t remaining) const {
        const int64_t a = opt_.prefill_chunk_alignment;
        if (a <= 1 || n <= 0 || n >= remaining) return n;
        const int64_t end = (computed + n) / a * a;
        return end > computed ? end - computed : 0;
    }

    // Rows of logits a step has beyond one per request.
    int64_t spare_rows() const {
        return opt_.max_logits_rows > opt_.max_num_seqs ? opt_.max_logits_rows - opt_.max_num_seqs : 0;
    }
    // The prompt positions of [c, c + n) at which r still wants logits: [first, second).
    static std::pair<int64_t, int64_t> prompt_rows(const Request& r, int64_t c, int64_t n) {
        if (!r.every_row) return {0, 0};
        const int64_t lo = std::max<int64_t>(c, r.rows_done), hi = std::min<int64_t>(c + n, r.num_prompt - 1);
        return hi > lo ? std::make_pair(lo, hi) : std::make_pair<int64_t, int64_t>(0, 0);
    }
    // The most of n tokens from c on whose prompt rows fit into `spare`.
    static int64_t fit_rows(const Request& r, int64_t c, int64_t n, int64_t spare) {
        const auto rows = prompt_rows(r, c, n);
        return rows.second - rows.first <= spare ? n : rows.first + spare - c;
    }

    // ---- one step
    const StepPlan& schedule() {
        if (plan_.open || prev_.open)
            throw Error(ERR_VALUE, "a planned step has not been updated (plan ahead with schedule_ahead)");
        return plan(false);
    }

    // ---- looking one step ahead (in the manner of crates/core/src/sched/mod.rs:8-9,646-670,690-760: the next step
    // is planned and launched while the last one still runs, with a placeholder for the token it will bring) ----
    // Only the plain case is taken ahead: the running step feeds one token of every request and samples each, nobody
    // waits, and every cache group has a free page for every running request, so the step ahead is "everyone decodes
    // once more" and preempts nobody. Anything else is planned after the running step's update, as before.
    bool can_look_ahead() const {
        if (!plan_.open || prev_.open || !waiting_.empty() || plan_.scheduled.empty()) return false;
        // a running request the step left out (no budget for it, a portion that could not be aligned) would come into
        // the step ahead with a token the host already knows, where every row is taken to wait for the running step
        if (plan_.scheduled.size() != running_.size()) return false;
        for (const Scheduled& s : plan_.scheduled)
            if (s.num_new != 1 || !s.samples) return false;
        for (int g = 0; g < cache_->num_groups(); ++g)
            if (cache_->pool(g).num_free() < static_cast<int64_t>(running_.size())) return false;
        return true;
    }

    const StepPlan& schedule_ahead() {
        if (!can_look_ahead()) throw Error(ERR_VALUE, "this step cannot be planned ahead");
        prev_ = std::move(plan_);
        plan_ = StepPlan{};
        int32_t k = 0;
        for (const Scheduled& s : prev_.scheduled) {
            const int32_t at = k++;  // every row of the running step samples
            auto it = reqs_.find(s.id);
            if (it == reqs_.end() || it->second->status != RUNNING) continue;
            Request* r = it->second.get();
            if (r->num_output() + 1 >= r->max_tokens || r->num_tokens() + 1 >= opt_.max_model_len) {
                r->ending = true;
                continue;
            }
            r->tokens.push_back(-1);
            r->pending = 1;
            r->pending_src = at;
        }
        return plan(true);
    }

private:
    const StepPlan& plan(bool ahead) {
        plan_.scheduled.clear();
        plan_.preempted.clear();
        plan_.force_finished.clear();
        plan_.feedback.clear();
        int64_t budget = opt_.max_num_batched_tokens;
        int64_t quota = opt_.prefill_tokens_per_step > 0 ? opt_.prefill_tokens_per_step : (int64_t(1) << 62);
        const size_t eligible = running_.size() + waiting_.size();
        const int64_t threshold = eligible > 1 ? opt_.long_prefill_token_threshold : 0;
        bool preempted_any = false;
        int64_t spare = spare_rows();
        auto put = [&](Request* r, int64_t n, int32_t feedback) {
            const auto rows = prompt_rows(*r, r->num_computed, n);
            plan_.scheduled.push_back({r->id, r->num_computed, static_cast<int32_t>(n),
                                       r->num_computed + n == r->num_tokens(), static_cast<int32_t>(rows.first),
                                       static_cast<int32_t>(rows.second - rows.first)});
            plan_.feedback.push_back(feedback);
            spare -= rows.second - rows.first;
        };

        size_t i = 0;
        while (i < running_.size()) {
            Request* r = running_[i];
            if (r->ending) {  // its last token is on its way
                ++i;
                continue;
            }
            const int64_t remaining = r->num_tokens() - r->num_computed;
            const bool is_decode = remaining == 1 && r->num_computed > 0;
            const bool charged = !(opt_.decode_exempt_from_budget && is_decode);
            if (charged && budget == 0) break;
            int64_t n = remaining;
            if (threshold && n > threshold) n = threshold;
            if (charged) n = std::min(n, budget);
            if (!is_decode) n = std::min(n, quota);
            n = fit_rows(*r, r->num_computed, n, spare);
            if (n < remaining && !opt_.enable_chunked_prefill) n = 0;
            n = aligned(r->num_computed, n, remaining);
            if (n <= 0) {
                ++i;
                continue;
            }
            bool got = false;
            for (;;) {
                if (cache_->allocate(r->id, r->num_computed, n)) {
                    got = true;
                    break;
                }
                if (ahead) break;  // the running step reads everyone's pages: nobody is preempted under it
                Request* victim = running_.back();
                if (victim == r) {
                    if (running_.size() > 1) break;  // others hold the pages; try again next step, never preempt oneself
                    finish(r, LENGTH);               // alone and still no page: the pool cannot hold it
                    plan_.force_finished.emplace_back(r->id, LENGTH);
                    break;
                }
                running_.pop_back();
                preempt(victim);
                plan_.preempted.push_back(victim->id);
                preempted_any = true;
            }
            if (!got) break;
            put(r, n, r->pending && r->num_computed + n == r->num_tokens() ? r->pending_src : -1);
            if (charged) budget -= n;
            if (!is_decode) quota -= n;
            ++i;
        }

        if (!preempted_any && !ahead) {
            while (budget > 0 && !waiting_.empty() && static_cast<int>(running_.size()) < opt_.max_num_seqs) {
                Request* r = waiting_.front();
                if (!cache_->can_admit()) break;
                cache_->admit(r->id);
                // a prefix of the prompt (or, after a preemption, of prompt and outputs) may be in the cache
                // still: those tokens are not computed again (:564-570)
                const bool rows_open = r->every_row && r->rows_done < r->num_prompt - 1;  // every position is computed
                if (opt_.enable_prefix_caching && r->num_computed == 0 && !rows_open) {
                    r->num_cached = static_cast<int32_t>(cache_->lookup(r->id, r->tokens.data(), r->num_tokens()));
                    r->num_computed = r->num_cached;
                }
                const int64_t remaining = r->num_tokens() - r->num_computed;
                int64_t n = remaining;
                if (threshold && n > threshold) n = threshold;
                n = std::min(n, std::min(budget, quota));
                n = fit_rows(*r, r->num_computed, n, spare);
                if (n < remaining && !opt_.enable_chunked_prefill) n = 0;
                n = aligned(r->num_computed, n, remaining);
                if (n <= 0 || !cache_->allocate(r->id, r->num_computed, n)) {
                    cache_->free(r->id);  // no budget or no pages now: wait (what was found stays cached)
                    if (opt_.enable_prefix_caching) r->num_computed = r->num_cached = 0;
                    break;
                }
                waiting_.pop_front();
                r->status = RUNNING;
                running_.push_back(r);
                put(r, n, -1);
                budget -= n;
                quota -= n;
            }
        }
        // advance at once, as the reference does after scheduling (:646-670)
        for (const Scheduled& s : plan_.scheduled) {
            Request* r = reqs_.at(s.id).get();
            if (r->status == RUNNING) r->num_computed = s.start + s.num_new;
            if (s.num_rows > 0) r->rows_done = s.rows_from + s.num_rows;
        }
        plan_.open = !plan_.scheduled.empty();
        return plan_;
    }

public:

    // sampled: one token for every scheduled request that samples, in the plan's order; of the oldest plan that is
    // not updated yet (the running step's, where the next one was planned ahead).
    // Appends one result for every scheduled request that is still running.
    void update(const int32_t* sampled, int n_sampled, std::vector<UpdateResult>& results) {
        StepPlan& p = prev_.open ? prev_ : plan_;
        if (!p.open) return;  // an empty plan, or one that was updated already: nothing to apply
        p.open = false;
        int k = 0;
        for (const Scheduled& s : p.scheduled) {
            const int at = s.samples ? k++ : -1;
            auto it = reqs_.find(s.id);
            if (it == reqs_.end() || it->second->status != RUNNING) continue;  // preempted, aborted or ended meanwhile
            Request* r = it->second.get();
            int32_t tok = -1;
            Reason reason = NO_REASON;
            if (s.samples) {
                if (at >= n_sampled) throw Error(ERR_VALUE, "fewer sampled tokens than sampling requests");
                tok = sampled[at];
                if (r->pending) {  // the step ahead was planned around this token: its placeholder gets its value
                    r->tokens.back() = tok;
                    r->pending = 0;
                    r->pending_src = -1;
                } else {
                    r->tokens.push_back(tok);
                }
                reason = check_stop(*r, tok);
            }
            // (the tokens counted as computed may include the one a step ahead is computing now: what is released
            // or committed here is used again only by steps launched later, which run after it)
            cache_->release_passed(r->id, r->num_computed);
            if (opt_.enable_prefix_caching) cache_->commit(r->id, r->tokens.data(), r->num_computed);
            if (reason != NO_REASON) finish(r, reason);
            results.push_back({r->id, tok, reason});
        }
    }

    // The plan's entries over the requests' own token storage (valid until the next update).
    void plan_entries(std::vector<EntryView>& entries, std::vector<int32_t>& want_store) const {
        entries.clear();
        size_t rows = 0;
        for (const Scheduled& s : plan_.scheduled) rows += s.num_rows;
        want_store.assign(plan_.scheduled.size() + rows, 0);  // (sized once: the entries point into it)
        size_t i = 0, at = plan_.scheduled.size();
        for (const Scheduled& s : plan_.scheduled) {
            const Request* r = reqs_.at(s.id).get();
            want_store[i] = s.num_new - 1;
            for (int32_t j = 0; j < s.num_rows; ++j) want_store[at + j] = s.rows_from - s.start + j;
            entries.push_back({s.id, s.start, s.num_new, r->tokens.data() + s.start, &want_store[i], s.samples ? 1 : 0,
                               plan_.feedback[i], &want_store[at], s.num_rows});
            at += s.num_rows;
            ++i;
        }
    }

private:
    Reason check_stop(const Request& r, int32_t tok) const {
        if (r.num_output() >= r.min_tokens) {
            if (!r.ignore_eos && eos_.count(tok)) return STOP;
            if (std::find(r.stop_ids.begin(), r.stop_ids.end(), tok) != r.stop_ids.end()) return STOP;
        }
        if (r.num_tokens() >= opt_.max_model_len || r.num_output() >= r.max_tokens) return LENGTH;
        return NO_REASON;
    }

    void preempt(Request* r) {
        cache_->free(r->id);
        r->num_computed = 0;
        r->status = PREEMPTED;
        ++r->preemptions;
        waiting_.push_front(r);
    }

    void finish(Request* r, Reason reason) {
        if (r->status == FINISHED) return;
        if (cache_->has(r->id)) cache_->free(r->id);
        running_.erase(std::remove(running_.begin(), running_.end(), r), running_.end());
        waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), r), waiting_.end());
        r->status = FINISHED;
        r->reason = reason;
    }

    SchedOptions opt_;
    CacheManager* cache_;
    std::unordered_set<int32_t> eos_;
    std::deque<Request*> waiting_;
    std::vector<Request*> running_;
    std::unordered_map<int64_t, std::unique_ptr<Request>> reqs_;
    StepPlan plan_;  // the newest plan
    StepPlan prev_;  // the plan before it while that one's step still runs (open), else spent
};

}  // namespace dinfer
