"""The scheduler's decisions (no GPU), driven step by step with made-up sampled tokens. The vectors
are the ones the reference's own tests hold (crates/core/src/sched/mod.rs:830-1442)."""
import pytest

from dinfer_amd.cache import CacheManager, GroupSpec
from dinfer_amd.config import EngineOptions
from dinfer_amd.engine.request import LENGTH, PREEMPTED, STOP, Request
from dinfer_amd.engine.scheduler import Scheduler
from dinfer_amd.sampling import SamplingParams


def mk(max_seqs, budget, blocks, **kw):
    kw = {"max_model_len": 4096, "decode_exempt_from_budget": False, **kw}
    opt = EngineOptions(max_num_seqs=max_seqs, max_num_batched_tokens=budget, block_size=16, num_blocks=blocks, **kw)
    cache = CacheManager([GroupSpec(16, blocks)], max_seqs)
    return Scheduler(opt, cache, eos_token_ids=[2])


def req(i, prompt, max_tokens, **kw):
    base = 100 + i * 10_000
    return Request(i, list(range(base, base + prompt)), SamplingParams(max_tokens=max_tokens, **kw))


def step(s, toks):
    """One schedule + update; toks: {id: sampled token} for the requests expected to sample."""
    out = s.schedule()
    assert {x.request.id for x in out.scheduled if x.samples} == set(toks)
    res = s.update(out, toks)
    s.cache.check()
    return [(x.request.id, x.num_new) for x in out.scheduled], out, res


def test_prefill_then_decode_then_finish_by_eos():
    s = mk(8, 64, 32)
    s.add_request(req(1, 10, 100))
    assert step(s, {1: 7})[0] == [(1, 10)]
    free = s.cache.num_free()
    assert step(s, {1: 8})[0] == [(1, 1)]
    assert s.cache.num_free() == free               # a decode inside the last page takes no page
    sched, _, res = step(s, {1: 2})
    assert res[0][1:] == (2, STOP) and not s.has_unfinished() and s.cache.num_free() == 32


def test_chunked_prefill_splits_by_budget():
    s = mk(8, 32, 64)
    s.add_request(req(1, 70, 4))
    assert step(s, {})[0] == [(1, 32)]
    assert step(s, {})[0] == [(1, 32)]
    assert step(s, {1: 9})[0] == [(1, 6)]           # the last portion samples
    assert step(s, {1: 9})[0] == [(1, 1)]


def test_fcfs_second_request_waits_for_budget_then_runs_alongside():
    s = mk(8, 40, 64)
    s.add_request(req(1, 30, 10))
    s.add_request(req(2, 30, 10))
    assert step(s, {1: 1})[0] == [(1, 30), (2, 10)]
    assert step(s, {1: 1, 2: 1})[0] == [(1, 1), (2, 20)]
    assert step(s, {1: 1, 2: 1})[0] == [(1, 1), (2, 1)]


def test_preempts_last_running_when_out_of_blocks_and_replays_everything():
    s = mk(8, 1000, 4)                               # 4 pages = 64 tokens: two 32-token prompts fill it
    s.add_request(req(1, 32, 2))
    r2 = req(2, 32, 100)
    s.add_request(r2)
    assert len(step(s, {1: 1, 2: 1})[0]) == 2
    sched, out, _ = step(s, {1: 1})                  # both need a third page: 1 gets it, 2 is preempted
    assert sched == [(1, 1)] and out.preempted == [2]
    assert r2.status == PREEMPTED and r2.num_computed == 0 and list(s.waiting) == [r2]
    assert 1 not in s.requests                       # request 1 reached max_tokens and freed its pages
    assert step(s, {2: 5})[0] == [(2, 33)]           # replays the prompt and its one output
    assert r2.output_ids == [1, 5]


def test_step_that_preempted_admits_nobody():
    s = mk(8, 1000, 4)
    s.add_request(req(1, 32, 100))
    s.add_request(req(2, 32, 100))
    step(s, {1: 1, 2: 1})
    s.add_request(req(3, 4, 100))
    sched, out, _ = step(s, {1: 1})
    assert sched == [(1, 1)] and out.preempted == [2] and [r.id for r in s.waiting] == [2, 3]


def test_decode_exempt_from_budget_coschedules_decode_and_prefill():
    s = mk(4, 8, 64, decode_exempt_from_budget=True)
    s.add_request(req(1, 4, 16))
    assert step(s, {1: 1})[0] == [(1, 4)]
    s.add_request(req(2, 20, 16))
    assert step(s, {1: 1})[0] == [(1, 1), (2, 8)]    # the decode row is free, the prompt gets all 8
    s2 = mk(4, 8, 64)
    s2.add_request(req(1, 4, 16))
    step(s2, {1: 1})
    s2.add_request(req(2, 20, 16))
    assert step(s2, {1: 1})[0] == [(1, 1), (2, 7)]   # charged: only 7 are left


def test_sole_request_that_cannot_grow_is_finished_with_length():
    s = mk(8, 1000, 4)
    r = req(1, 48, 100)
    s.add_request(r)
    assert step(s, {1: 1})[0] == [(1, 48)]
    forced = []
    for _ in range(40):
        out = s.schedule()
        forced += out.force_finished
        if not out.scheduled:
            break
        s.update(out, {1: 1})
    assert forced == [(1, LENGTH)] and r.finish_reason == LENGTH and r.num_computed == 64  # 4 pages full
    assert s.cache.num_free() == 4 and not s.has_unfinished()


def test_tail_request_with_others_present_is_skipped_not_finished():
    s = mk(8, 1000, 6)                               # 6 pages: two 48-token prompts fill them
    s.add_request(req(1, 48, 2))
    r2 = req(2, 48, 100)
    s.add_request(r2)
    assert len(step(s, {1: 1, 2: 1})[0]) == 2
    sched, out, _ = step(s, {1: 1})
    assert sched == [(1, 1)] and r2.status == PREEMPTED and not out.force_finished
    sched, out, _ = step(s, {2: 1})                  # request 1 is done; 2 comes back and recomputes
    assert sched[0][0] == 2 and not out.force_finished


def test_waiting_request_without_pages_waits():
    s = mk(8, 1000, 3)
    s.add_request(req(1, 40, 100))
    s.add_request(req(2, 20, 100))
    assert step(s, {1: 1})[0] == [(1, 40)]           # 3 pages taken; request 2 needs 2
    assert [r.id for r in s.waiting] == [2]
    assert step(s, {1: 1})[0] == [(1, 1)]
    s.abort(1)
    assert step(s, {2: 1})[0] == [(2, 20)]


def test_finish_reasons():
    s = mk(8, 1000, 32)
    s.add_request(req(1, 4, 2))
    step(s, {1: 5})
    assert step(s, {1: 6})[2][0][2] == LENGTH        # max_tokens (mod.rs:1188-1195)
    s.add_request(req(2, 4, 10, ignore_eos=True))
    assert step(s, {2: 2})[2][0][2] is None          # eos ignored
    s.add_request(req(3, 4, 10, stop_token_ids=[77]))
    res = step(s, {2: 2, 3: 77})[2]
    assert dict((r.id, why) for r, _, why in res) == {2: None, 3: STOP}
    s.add_request(req(4, 4, 10, min_tokens=3))
    assert step(s, {2: 9, 4: 2})[2][-1][2] is None   # eos before min_tokens does not stop
    step(s, {2: 9, 4: 2})
    assert step(s, {2: 9, 4: 2})[2][-1][2] == STOP


def test_max_model_len_finishes_with_length():
    s = mk(8, 1000, 32, max_model_len=8)
    s.add_request(req(1, 6, 100))
    step(s, {1: 5})
    assert step(s, {1: 5})[2][0][2] == LENGTH        # 8 tokens reached
    import pytest
    with pytest.raises(ValueError, match="max_model_len"):
        s.add_request(req(2, 8, 1))


def test_per_request_and_per_step_prompt_caps():
    s = mk(8, 1000, 64, long_prefill_token_threshold=8)
    s.add_request(req(1, 30, 4))
    assert step(s, {1: 1})[0] == [(1, 30)]           # alone: the cap does not apply (mod.rs:343-346)
    s.add_request(req(2, 30, 4))
    s.add_request(req(3, 30, 4))
    assert step(s, {1: 1})[0] == [(1, 1), (2, 8), (3, 8)]
    s = mk(8, 1000, 64, prefill_tokens_per_step=10)
    s.add_request(req(1, 6, 4))
    s.add_request(req(2, 30, 4))
    assert step(s, {1: 1})[0] == [(1, 6), (2, 4)]    # 10 prompt tokens per step over all requests
    assert step(s, {1: 1})[0] == [(1, 1), (2, 10)]   # decode rows are outside the quota


def test_max_num_seqs_limits_admission():
    s = mk(2, 1000, 64)
    for i in (1, 2, 3):
        s.add_request(req(i, 4, 1))
    assert [i for i, _ in step(s, {1: 1, 2: 1})[0]] == [1, 2]
    assert step(s, {3: 1})[0] == [(3, 4)]


def test_schedule_and_update_are_cheap_for_many_decode_rows():
    """The reference gates 1024 decode requests at 200 us (crates/core/benches/scheduler.rs). The
    decisions here are C++ too, but this gate times the Python front with them (one object per
    request and step), so it is wider: 256 decode rows within 1 ms."""
    import time
    n = 256
    s = mk(n, 100000, n * 4)
    for i in range(n):
        s.add_request(req(i, 17, 1000))
    out = s.schedule()
    s.update(out, {i: 1 for i in range(n)})
    t0 = time.perf_counter()
    for _ in range(10):
        out = s.schedule()
        s.update(out, {i: 1 for i in range(n)})
    assert (time.perf_counter() - t0) / 10 < 0.001


def test_random_loads_keep_every_rule():
    """Random prompts, limits and arrival times against a tight pool: every step obeys the budget and
    the request limit, only the last running request is ever preempted, nothing is lost in the cache,
    and every request ends with exactly the outputs it was allowed."""
    import random
    preemptions = 0
    for seed in range(6):
        rng = random.Random(seed)
        budget, max_seqs, blocks = rng.choice([8, 24, 64]), rng.choice([2, 3, 5]), rng.choice([6, 9, 14])
        s = mk(max_seqs, budget, blocks, decode_exempt_from_budget=bool(seed % 2), max_model_len=blocks * 16)
        todo = [req(i, rng.randrange(1, 60), rng.randrange(1, 30)) for i in range(12)]
        todo = [r for r in todo if r.num_prompt + r.sampling.max_tokens <= blocks * 16 - 16]
        everyone = list(todo)
        steps = 0
        while todo or s.has_unfinished():
            steps += 1
            assert steps < 5000
            while todo and rng.random() < 0.4:
                s.add_request(todo.pop())
            running_before = [r.id for r in s.running]
            out = s.schedule()
            charged = sum(x.num_new for x in out.scheduled
                          if not (s.opt.decode_exempt_from_budget and x.num_new == 1 and x.start > 0))
            assert charged <= budget and len(s.running) <= max_seqs
            assert out.preempted == running_before[len(running_before) - len(out.preempted):][::-1]
            preemptions += len(out.preempted)
            for x in out.scheduled:
                assert x.start + x.num_new <= x.request.num_tokens and x.samples == (x.start + x.num_new == x.request.num_tokens)
            s.update(out, {x.request.id: 3 for x in out.scheduled if x.samples})
            s.cache.check()
        for r in everyone:
            assert r.status == "finished" and r.finish_reason == LENGTH and r.num_output == r.sampling.max_tokens, r
        assert s.cache.num_free() == blocks and not s.requests
    assert preemptions > 10


# ---- prefix caching ---------------------------------------------------------------------------------
def mkp(max_seqs, budget, blocks, **kw):
    kw = {"max_model_len": 4096, "decode_exempt_from_budget": False, "enable_prefix_caching": True, **kw}
    opt = EngineOptions(max_num_seqs=max_seqs, max_num_batched_tokens=budget, block_size=16, num_blocks=blocks, **kw)
    cache = CacheManager([GroupSpec(16, blocks)], max_seqs, prefix_caching=True)
    return Scheduler(opt, cache, eos_token_ids=[2])


def same_prompt(i, n, max_tokens):
    return Request(i, list(range(500, 500 + n)), SamplingParams(max_tokens=max_tokens))


def test_second_request_with_the_same_prompt_skips_the_cached_pages():
    """sched/mod.rs:564-570 with kv/manager.rs:150-199: 40 tokens, pages of 16: the second request finds
    32 tokens cached and feeds 8."""
    s = mkp(4, 100, 16)
    r1, r2 = same_prompt(1, 40, 3), same_prompt(2, 40, 2)
    s.add_request(r1)
    assert step(s, {1: 7})[0] == [(1, 40)]
    s.add_request(r2)
    sched, out, _ = step(s, {1: 7, 2: 7})
    assert sched == [(1, 1), (2, 8)] and out.scheduled[1].start == 32
    assert r2.num_cached_tokens == 32 and r1.num_cached_tokens == 0
    t1, t2 = s.cache.block_table(1, 0), s.cache.block_table(2, 0)
    assert t1[:2] == t2[:2] and t1[2] != t2[2]
    step(s, {1: 7, 2: 7})
    assert not s.has_unfinished() and s.cache.num_free() == 16


def test_a_prompt_that_is_cached_whole_still_computes_its_last_token():
    s = mkp(4, 100, 16)
    s.add_request(same_prompt(1, 32, 1))
    step(s, {1: 7})
    r2 = same_prompt(2, 32, 1)
    s.add_request(r2)
    sched, out, _ = step(s, {2: 7})
    assert sched == [(2, 16)] and out.scheduled[0].start == 16 and r2.num_cached_tokens == 16


def test_preempted_request_finds_its_own_pages_again():
    """Without a prefix cache a preempted request replays everything (sched/mod.rs:979-991); with it, the
    pages that were not handed out meanwhile are still there."""
    s = mkp(4, 100, 5)
    r1, r2 = req(1, 32, 20), req(2, 31, 40)
    s.add_request(r1)
    s.add_request(r2)
    assert step(s, {1: 5, 2: 5})[0] == [(1, 32), (2, 31)]          # pages 0, 1 and 2, 3; page 4 is free
    assert step(s, {1: 5, 2: 5})[0] == [(1, 1), (2, 1)]            # request 1 takes page 4, request 2 fills page 3
    # request 2 needs a page and is the last one running: it is skipped while request 1 goes on ...
    for _ in range(15):
        sched, out, _ = step(s, {1: 5})
        assert sched == [(1, 1)] and not out.preempted
    # ... until request 1 needs a page itself: request 2 is preempted, its two full pages go to the tail
    sched, out, _ = step(s, {1: 5})
    assert sched == [(1, 1)] and out.preempted == [2] and r2.num_computed == 0
    while r1.status != "finished":
        step(s, {1: 5})
    # request 1 took the younger of the two pages (the tail of request 2 is evicted first); the other is found again
    sched, out, _ = step(s, {2: 5})
    assert sched == [(2, 33 - 16)] and out.scheduled[0].start == 16 and r2.num_cached_tokens == 16
    assert r2.num_preemptions == 1


def test_random_loads_with_prefix_caching_keep_every_rule():
    import random
    cached = 0
    for seed in range(6):
        rng = random.Random(100 + seed)
        budget, max_seqs, blocks = rng.choice([8, 24, 64]), rng.choice([2, 3, 5]), rng.choice([8, 12, 20])
        s = mkp(max_seqs, budget, blocks, decode_exempt_from_budget=bool(seed % 2), max_model_len=blocks * 16)
        stems = [[rng.randrange(1000) + 10 for _ in range(70)] for _ in range(2)]
        todo = []
        for i in range(14):
            p = rng.choice(stems)[:rng.randrange(1, 60)] + [rng.randrange(1000) + 10 for _ in range(rng.randrange(0, 4))]
            mt = rng.randrange(1, 20)
            if len(p) + mt <= blocks * 16 - 16:
                todo.append(Request(i, p, SamplingParams(max_tokens=mt)))
        everyone = list(todo)
        steps = 0
        while todo or s.has_unfinished():
            steps += 1
            assert steps < 5000
            while todo and rng.random() < 0.4:
                s.add_request(todo.pop())
            out = s.schedule()
            charged = sum(x.num_new for x in out.scheduled
                          if not (s.opt.decode_exempt_from_budget and x.num_new == 1 and x.start > 0))
            assert charged <= budget and len(s.running) <= max_seqs
            for x in out.scheduled:
                assert x.num_new >= 1 and x.samples == (x.start + x.num_new == x.request.num_tokens)
            s.update(out, {x.request.id: 3 for x in out.scheduled if x.samples})
            s.cache.check()
        for r in everyone:
            assert r.status == "finished" and r.num_output == r.sampling.max_tokens, r
            cached += r.num_cached_tokens
        assert s.cache.num_free() == blocks and not s.requests
    assert cached > 200


def test_request_ids_can_be_used_again_and_aborts_free_everything():
    s = mk(4, 100, 16)
    a = req(1, 20, 5)
    s.add_request(a)
    import pytest
    with pytest.raises(KeyError):
        s.add_request(req(1, 3, 1))                  # the id is live
    step(s, {1: 9})
    s.abort(1)                                       # while running
    assert a.status == "finished" and a.finish_reason == "abort" and not s.has_unfinished()
    assert s.cache.num_free() == 16 and not s.cache.has(1)
    b = req(1, 7, 2)                                 # the same id again, a different request
    s.add_request(b)
    s.add_request(req(2, 5, 2))
    s.abort(2)                                       # while waiting
    assert [r.id for r in s.waiting] == [1]
    assert step(s, {1: 9})[0] == [(1, 7)] and b.num_computed == 7 and a.num_computed == 20
    s.abort(99)                                      # unknown: nothing happens
    step(s, {1: 9})
    assert not s.has_unfinished() and s.cache.num_free() == 16
    s.cache.check()


def test_abort_between_schedule_and_update_drops_the_sample():
    s = mk(4, 100, 16)
    s.add_request(req(1, 4, 5))
    s.add_request(req(2, 4, 5))
    out = s.schedule()
    s.abort(1)
    res = s.update(out, {1: 7, 2: 8})                # the token for request 1 is ignored
    assert [(r.id, t) for r, t, _ in res] == [(2, 8)]
    s.cache.check()
    assert s.cache.num_free() == 15


def test_portions_end_at_multiples_of_the_alignment():
    """With an alignment of 16 every portion that does not end its request's tokens ends at a multiple of 16: the
    budget of 40 gives 32; what is left of it (8) is no aligned portion for the second request, which waits; the
    last portion of a prompt may end anywhere; decoding is untouched."""
    s = mk(8, 40, 64, prefill_chunk_alignment=16)
    s.add_request(req(1, 70, 3))
    s.add_request(req(2, 21, 3))
    assert step(s, {})[0] == [(1, 32)]                       # 40 cut back to 32; 8 left: less than one aligned portion of 2
    assert step(s, {1: 9})[0] == [(1, 38)]                   # ends the prompt: may end anywhere; 2 left, nothing for 2
    assert step(s, {1: 9, 2: 9})[0] == [(1, 1), (2, 21)]     # a whole prompt needs no alignment either
    assert step(s, {1: 9, 2: 9})[0] == [(1, 1), (2, 1)]
    s = mk(8, 20, 64, prefill_chunk_alignment=16, long_prefill_token_threshold=24)
    s.add_request(req(1, 50, 2))
    s.add_request(req(2, 50, 2))
    sched = step(s, {})[0]
    assert sched == [(1, 16)]                                # 20 -> 16; the 4 left hold no aligned portion
    assert step(s, {})[0] == [(1, 16)]


# ---- planning one step ahead (crates/core/src/sched/mod.rs:8-9,646-670,690-760: placeholders for tokens on their way) ----
def ahead_run(s, tokens_of, steps):
    """Drives s with one step always planned ahead where that is allowed. tokens_of(request id, its output count)
    gives the token a step samples. Returns {id: outputs} and how many steps were planned ahead."""
    got, running, ahead_count = {}, None, 0
    for _ in range(steps):
        if running is None:
            out = s.schedule()
            if not len(out):
                if not s.has_unfinished():
                    break
                continue
            running = out
        nxt = None
        if s.can_look_ahead():
            nxt = s.schedule(ahead=True)
            ahead_count += 1
            assert all(x.num_new == 1 and x.samples for x in nxt.scheduled) and not nxt.preempted
            nxt = nxt if len(nxt) else None
        toks = {r.id: tokens_of(r.id, len(got.get(r.id, []))) for r in running.sampling_requests()}
        for r, tok, reason in s.update(running, toks):
            if tok is not None:
                got.setdefault(r.id, []).append(tok)
        s.cache.check()
        running = nxt
    return got, ahead_count


def plain_run(s, tokens_of, steps):
    got = {}
    for _ in range(steps):
        if not s.has_unfinished():
            break
        out = s.schedule()
        toks = {r.id: tokens_of(r.id, len(got.get(r.id, []))) for r in out.sampling_requests()}
        for r, tok, reason in s.update(out, toks):
            if tok is not None:
                got.setdefault(r.id, []).append(tok)
    return got


def test_a_step_planned_ahead_feeds_the_token_that_is_on_its_way():
    s = mk(8, 64, 32)
    r1 = req(1, 10, 100)
    s.add_request(r1)
    out = s.schedule()
    assert not s.can_look_ahead()                      # a prompt portion runs: not the plain case
    s.update(out, {1: 7})
    out = s.schedule()                                 # the first decode step, planned after its input was known
    assert [(x.start, x.num_new) for x in out.scheduled] == [(10, 1)] and s.can_look_ahead()
    nxt = s.schedule(ahead=True)
    assert [(x.start, x.num_new, x.samples) for x in nxt.scheduled] == [(11, 1, True)]
    assert s.request_info(r1).num_tokens == 12          # prompt, one output, one placeholder
    assert not s.can_look_ahead()                       # two steps are out already
    res = s.update(out, {1: 8})                         # the running step's token fills the placeholder
    assert [(r.id, t, why) for r, t, why in res] == [(1, 8, None)] and r1.output_ids == [7, 8]
    assert s.request_info(r1).num_tokens == 12
    assert s.can_look_ahead()                           # now the plan ahead is the running one
    res = s.update(nxt, {1: 9})
    assert r1.output_ids == [7, 8, 9] and s.request_info(r1).num_tokens == 13
    s.cache.check()


def test_planned_ahead_gives_the_same_tokens_and_ends_as_step_by_step():
    def tokens_of(rid, n):                              # request 2 meets the end-of-sequence token as its 6th
        return 2 if (rid == 2 and n == 5) else 10 + rid + n
    runs = []
    for drive in (plain_run, lambda s, t, n: ahead_run(s, t, n)[0]):
        s = mk(8, 64, 64)
        for i, (plen, mx) in enumerate([(10, 9), (20, 30), (5, 4)], start=1):
            s.add_request(req(i, plen, mx))
        runs.append(drive(s, tokens_of, 100))
        assert not s.has_unfinished() and s.cache.num_free() == 64
        s.cache.check()
    assert runs[0] == runs[1]
    assert len(runs[0][1]) == 9 and runs[0][2][-1] == 2 and len(runs[0][2]) == 6 and len(runs[0][3]) == 4


def test_a_request_that_ends_unforeseen_leaves_a_row_nobody_waits_for():
    s = mk(8, 64, 32)
    r1, r2 = req(1, 10, 100), req(2, 10, 100)
    s.add_request(r1)
    s.add_request(r2)
    s.update(s.schedule(), {1: 5, 2: 5})
    run = s.schedule()
    nxt = s.schedule(ahead=True)
    assert [x.request.id for x in nxt.scheduled] == [1, 2]
    res = s.update(run, {1: 2, 2: 6})                   # request 1 samples the end-of-sequence token
    assert [(r.id, why) for r, _, why in res] == [(1, STOP), (2, None)] and 1 not in s.requests
    free = s.cache.num_free()
    res = s.update(nxt, {1: 99, 2: 7})                  # its row in the step ahead was computed in vain
    assert [(r.id, t) for r, t, _ in res] == [(2, 7)] and r1.output_ids == [5, 2] and r2.output_ids == [5, 6, 7]
    assert s.cache.num_free() == free
    s.cache.check()


def test_no_step_is_planned_ahead_for_the_last_token_of_a_request():
    s = mk(8, 64, 32)
    r1, r2 = req(1, 10, 2), req(2, 10, 100)
    s.add_request(r1)
    s.add_request(r2)
    s.update(s.schedule(), {1: 5, 2: 5})
    run = s.schedule()
    nxt = s.schedule(ahead=True)                        # request 1's second token is its last whatever it is
    assert [x.request.id for x in nxt.scheduled] == [2]
    res = s.update(run, {1: 6, 2: 6})
    assert [(r.id, why) for r, _, why in res] == [(1, LENGTH), (2, None)]
    s.update(nxt, {2: 7})
    assert r2.output_ids == [5, 6, 7]
    s.cache.check()


def test_nothing_is_planned_ahead_when_someone_waits_or_pages_are_short():
    s = mk(1, 64, 32)                                   # one request slot: the second request waits
    s.add_request(req(1, 10, 100))
    s.add_request(req(2, 10, 100))
    s.update(s.schedule(), {1: 5})
    s.schedule()
    assert not s.can_look_ahead()
    s = mk(8, 64, 3)                                    # three pages of 16: the prompts take two
    s.add_request(req(1, 16, 100))
    s.add_request(req(2, 15, 100))
    s.update(s.schedule(), {1: 5, 2: 5})
    out = s.schedule()                                  # request 1's decode takes the last free page
    assert [x.request.id for x in out.scheduled] == [1, 2] and not out.preempted and s.cache.num_free() == 0
    assert not s.can_look_ahead()                       # a step ahead might have to preempt: it waits


def test_nothing_is_planned_ahead_while_a_running_request_is_left_out_of_the_step():
    """A request in mid-prompt whose next portion cannot end at an aligned position is left out of a step; the step
    then holds one decoding row only, but not everyone who runs is in it: a step planned ahead would take "every
    row waits for the running step" for granted of a request that does not, so it is planned after the update."""
    s = mk(8, 20, 32, prefill_chunk_alignment=16, long_prefill_token_threshold=10)
    s.add_request(req(2, 40, 100))
    out = s.schedule()                                  # alone: no threshold, 20 tokens cut to the aligned 16
    assert [(x.request.id, x.num_new) for x in out.scheduled] == [(2, 16)]
    s.update(out, {})
    s.add_request(req(1, 1, 100))
    out = s.schedule()                                  # two are eligible: portions of 10 at most, none ends at 32
    assert [(x.request.id, x.num_new, x.samples) for x in out.scheduled] == [(1, 1, True)]
    assert not s.can_look_ahead()
    with pytest.raises(ValueError):
        s.schedule(ahead=True)
    s.update(out, {1: 7})
    s.cache.check()


def test_random_loads_planned_ahead_match_step_by_step():
    import random
    looked = 0
    for seed in range(6):
        rng = random.Random(seed)
        spec = [(rng.randrange(1, 60), rng.randrange(1, 40)) for _ in range(rng.randrange(2, 10))]
        stop_at = {i: rng.randrange(1, 40) for i in range(1, len(spec) + 1) if rng.random() < 0.4}
        tokens_of = lambda rid, n: 2 if stop_at.get(rid) == n else 10 + (rid * 31 + n * 7) % 1000
        blocks = rng.choice([8, 16, 64])
        # the same engine sizes for both ways of driving
        seqs, budget = rng.choice([2, 4, 8]), rng.choice([16, 64])
        outs = []
        for drive in (plain_run, ahead_run):
            s = mk(seqs, budget, blocks)
            for i, (plen, mx) in enumerate(spec, start=1):
                s.add_request(req(i, plen, mx))
            res = drive(s, tokens_of, 2000)
            outs.append(res if drive is plain_run else res[0])
            assert not s.has_unfinished() and s.cache.num_free() == blocks
            s.cache.check()
        assert outs[0] == outs[1], f"seed {seed}"
        looked += res[1]
    assert looked > 50                                  # the loads do spend most decode steps planned ahead


@pytest.mark.parametrize("fields,needle", [
    (dict(temperature=-0.1), "temperature"), (dict(top_p=0.0), "top_p"), (dict(top_k=0), "top_k"),
    (dict(min_p=1.5), "min_p"), (dict(repetition_penalty=0.0), "repetition_penalty"),
    (dict(frequency_penalty=2.5), "frequency_penalty"), (dict(presence_penalty=-2.5), "presence_penalty"),
    (dict(max_tokens=0), "max_tokens"), (dict(max_tokens=3, min_tokens=4), "min_tokens"),
    (dict(logprobs=21), "logprobs"), (dict(logprobs=-1), "logprobs"),
    (dict(logit_bias={5: 100.5}), "logit_bias"), (dict(logit_bias={-3: 1.0}), "logit_bias"),
    (dict(logit_bias={i: 0.5 for i in range(301)}), "at most 300"), (dict(seed=1 << 64), "seed")])
def test_sampling_options_out_of_range_are_refused_at_admission(fields, needle):
    """The ranges of crates/core/src/sample.rs:157-205."""
    s = mk(4, 64, 16)
    with pytest.raises(ValueError, match=needle):
        s.add_request(Request(0, [1, 2, 3], SamplingParams(**fields)))
    assert not s.has_unfinished()


def test_logit_bias_takes_a_mapping_or_pairs():
    a = SamplingParams(logit_bias={"7": 1, 9: -2.5})
    b = SamplingParams(logit_bias=[(7, 1.0), (9, -2.5)])
    assert a.logit_bias == b.logit_bias == {7: 1.0, 9: -2.5}
    a.validate()
    assert SamplingParams(logprobs=20, logit_bias={i: 100.0 for i in range(300)}).validate() is None
    with pytest.raises(ValueError, match="twice"):
        SamplingParams(logit_bias=[(7, 1.0), (7, 2.0)])
    assert SamplingParams(temperature=0.0).picks_largest_logit
    assert not SamplingParams(temperature=0.0, logit_bias={1: 1.0}).picks_largest_logit
    assert not SamplingParams(temperature=0.0, presence_penalty=0.5).picks_largest_logit


def rows_of(out):
    return [(x.request.id, x.start, x.num_new, bool(x.samples)) for x in out.scheduled], \
        [(r.id, p) for r, p in out.prompt_rows()]


def test_a_prompt_whose_every_position_is_wanted_is_cut_to_the_spare_rows():
    """prompt_logprobs: logits at every prompt position whose next token is in the prompt, at most as many a step
    as the engine has rows beyond one per request; the last prompt token's row is the sampling row."""
    s = mk(4, 64, 32, max_logits_rows=9)                       # 5 to spare
    s.add_request(req(1, 23, 3, prompt_logprobs=2))
    seen, cuts = [], []
    for _ in range(5):
        out = s.schedule()
        plan, rows = rows_of(out)
        cuts.append(plan[0][1:])
        seen += [p for _, p in rows]
        s.update(out, {1: 7} if plan[0][3] else {})
    assert cuts == [(0, 5, False), (5, 5, False), (10, 5, False), (15, 5, False), (20, 3, True)]
    assert seen == list(range(22))                           # each once, in order; position 22 samples
    out = s.schedule()
    assert rows_of(out) == ([(1, 23, 1, True)], [])          # decoding: nothing more


def test_two_such_prompts_share_the_spare_rows_and_others_are_not_held_up():
    s = mk(4, 64, 32, max_logits_rows=10)                      # 6 to spare
    s.add_request(req(1, 10, 2, prompt_logprobs=0))
    s.add_request(req(2, 30, 2))
    s.add_request(req(3, 10, 2, prompt_logprobs=0))
    # the first takes the six rows; the plain prompt between them goes in whole; the third finds no row left
    # and waits (and so does whoever comes after it)
    out = s.schedule()
    plan, rows = rows_of(out)
    assert plan == [(1, 0, 6, False), (2, 0, 30, True)] and rows == [(1, p) for p in range(6)]
    s.update(out, {2: 5})
    out = s.schedule()
    plan, rows = rows_of(out)
    assert plan == [(1, 6, 4, True), (2, 30, 1, True), (3, 0, 3, False)]
    assert rows == [(1, 6), (1, 7), (1, 8), (3, 0), (3, 1), (3, 2)]


def test_every_position_is_computed_whatever_the_prefix_cache_holds_and_once_whatever_is_preempted():
    cache = CacheManager([GroupSpec(16, 8)], 4, prefix_caching=True)
    opt = EngineOptions(max_num_seqs=4, max_num_batched_tokens=64, block_size=16, num_blocks=8, max_model_len=4096,
                        max_logits_rows=40, decode_exempt_from_budget=False)
    s = Scheduler(opt, cache, eos_token_ids=[2])
    first = Request(1, list(range(500, 540)), SamplingParams(max_tokens=1))
    s.add_request(first)
    s.update(s.schedule(), {1: 9})                           # ends; its two full pages stay in the prefix cache
    other = Request(3, list(range(900, 950)), SamplingParams(max_tokens=40))
    s.add_request(other)
    s.update(s.schedule(), {3: 7})
    same = Request(2, list(range(500, 540)), SamplingParams(max_tokens=30, prompt_logprobs=0))
    s.add_request(same)
    out = s.schedule()
    assert rows_of(out) == ([(3, 50, 1, True), (2, 0, 36, False)], [(2, p) for p in range(36)])
    assert same.num_cached_tokens == 0                       # (the same prompt without the option takes 32 from there)
    s.update(out, {3: 7})
    out = s.schedule()
    assert rows_of(out) == ([(3, 51, 1, True), (2, 36, 4, True)], [(2, 36), (2, 37), (2, 38)])
    s.update(out, {2: 7, 3: 7})
    # 4 + 3 pages of 8 are held; both decode until the first needs a page that is not there and the one admitted
    # last is preempted: when it comes back it computes its prompt again, and no position is reported twice
    seen = []
    for _ in range(200):
        out = s.schedule()
        seen += out.prompt_rows()
        s.update(out, {r.id: 7 for r in out.sampling_requests()})
        if not s.has_unfinished():
            break
    assert same.num_preemptions > 0 and seen == []
    assert same.finish_reason == other.finish_reason == "length" and same.num_output == 30


def test_every_position_needs_rows_to_spare():
    s = mk(4, 64, 32)
    with pytest.raises(ValueError, match="max_logits_rows"):
        s.add_request(req(1, 10, 2, prompt_logprobs=1))
    s = mk(4, 64, 32, max_logits_rows=8, enable_chunked_prefill=False)
    with pytest.raises(ValueError, match="spare rows"):
        s.add_request(req(1, 10, 2, prompt_logprobs=1))     # 9 rows, 4 to spare, and no cutting
    s.add_request(req(2, 5, 2, prompt_logprobs=1))          # 4 rows fit
    assert rows_of(s.schedule()) == ([(2, 0, 5, True)], [(2, 0), (2, 1), (2, 2), (2, 3)])
