"""The flat batch a step is built into (no GPU), against the exact plans the reference's runner tests
hold (crates/core/src/runner.rs:1058-1148), and the Engine loop with a stand-in runner."""
import numpy as np
import torch

from dinfer_amd.cache import CacheManager, GroupSpec
from dinfer_amd.config import EngineOptions
from dinfer_amd.engine.batch import Entry, StepBatch
from dinfer_amd.engine.request import Request
from dinfer_amd.engine.scheduler import Scheduler
from dinfer_amd.sampling import SamplingParams


def setup(budget):
    opt = EngineOptions(max_num_seqs=8, max_num_batched_tokens=budget, block_size=16, max_model_len=4096,
                        num_blocks=64, decode_exempt_from_budget=False)
    cache = CacheManager([GroupSpec(16, 64)], 8)
    return Scheduler(opt, cache, eos_token_ids=[]), StepBatch(torch.device("cpu"), 1024, 8, 8, [4])


def run(s, b):
    """schedule -> fill -> echo executor (token = 1000 + seq_len, runner.rs:888-905) -> update."""
    out = s.schedule()
    entries = [Entry(x.request.id, x.request.tokens(x.start, x.num_new), x.start, [x.num_new - 1] if x.samples else [])
               for x in out.scheduled]
    b.fill(entries, s.cache)
    sampled = {x.request.id: 1000 + x.start + x.num_new for x in out.scheduled if x.samples}
    s.update(out, sampled)
    return out


def test_two_requests_prefill_then_decode_then_finish():
    s, b = setup(1000)
    sp = lambda n: SamplingParams(max_tokens=n, temperature=0.0)
    r1, r2 = Request(1, list(range(20)), sp(3)), Request(2, list(range(5)), sp(2))
    s.add_request(r1)
    s.add_request(r2)
    run(s, b)
    h = b.h
    assert b.req_ids == [1, 2] and (b.num_tokens, b.num_reqs, b.num_rows) == (25, 2, 2)
    assert h["cu_seqlens"][:3].tolist() == [0, 20, 25] and h["logits_rows"][:2].tolist() == [19, 24]
    assert h["positions"][20:25].tolist() == [0, 1, 2, 3, 4]
    # request 1 holds pages 0, 1 and request 2 page 2: slot = page * 16 + offset
    assert h["slot_mapping0"][16] == 16 and h["slot_mapping0"][20] == 32
    assert h["block_table0"][:2, :2].tolist() == [[0, 1], [2, -1]]
    assert not b.all_decode and b.max_q_len == 20
    assert r1.output_ids == [1020] and r2.output_ids == [1005]
    run(s, b)   # two decode rows
    assert h["input_ids"][:2].tolist() == [1020, 1005] and h["positions"][:2].tolist() == [20, 5]
    assert h["seq_lens"][:2].tolist() == [21, 6] and h["slot_mapping0"][:2].tolist() == [20, 37]
    assert h["logits_rows"][:2].tolist() == [0, 1] and b.all_decode
    assert r2.finish_reason == "length"
    run(s, b)
    assert r1.finish_reason == "length" and r1.num_tokens == 23 and not s.has_unfinished()


def test_mixed_and_chunked_batches():
    s, b = setup(12)
    sp = SamplingParams(max_tokens=4, temperature=0.0)
    r1 = Request(1, list(range(20)), sp)
    s.add_request(r1)
    out = run(s, b)
    assert [(x.request.id, x.num_new) for x in out.scheduled] == [(1, 12)]
    assert b.num_rows == 0 and r1.output_ids == []          # a mid-prompt portion samples nothing
    r2 = Request(2, list(range(4)), sp)
    s.add_request(r2)
    out = run(s, b)
    assert [(x.request.id, x.num_new) for x in out.scheduled] == [(1, 8), (2, 4)]
    h = b.h
    assert h["cu_seqlens"][:3].tolist() == [0, 8, 12] and h["positions"][:8].tolist() == list(range(12, 20))
    assert h["seq_lens"][:2].tolist() == [20, 4] and h["logits_rows"][:2].tolist() == [7, 11]
    assert r1.output_ids == [1020] and r2.output_ids == [1004]
    run(s, b)
    assert b.all_decode and h["input_ids"][:2].tolist() == [1020, 1004]


def test_padding_for_a_graph_bucket():
    s, b = setup(1000)
    for i, n in ((1, 20), (2, 5), (3, 7)):
        s.add_request(Request(i, list(range(n)), SamplingParams(max_tokens=5)))
    run(s, b)
    out = s.schedule()
    entries = [Entry(x.request.id, x.request.tokens(x.start, 1), x.start, [0]) for x in out.scheduled]
    b.fill(entries, s.cache, pad_to=4)
    h = b.h
    assert (b.num_tokens, b.num_reqs, b.num_rows) == (4, 4, 4) and b.q_lens == [1, 1, 1, 1]
    assert h["cu_seqlens"][:5].tolist() == [0, 1, 2, 3, 4] and h["seq_lens"][:4].tolist() == [21, 6, 8, 1]
    assert h["slot_mapping0"][3] == -1 and h["block_table0"][3].tolist() == [0, 0, 0, 0]   # writes nothing, reads page 0
    assert h["logits_rows"][:4].tolist() == [0, 1, 2, 3]


def test_padding_a_step_with_portions_up_to_given_counts():
    """Made-up requests bring a step to the counts of a captured graph: one token each, the last one the rest; they
    write nothing (slot -1), hold page 0 everywhere and the spare state slot; made-up logits rows point at the first
    made-up token. What the real requests brought stays as it was."""
    import pytest
    s, b = setup(1000)
    s.cache.admit("x")
    s.cache.admit("y")
    assert s.cache.allocate("x", 0, 13) and s.cache.allocate("y", 0, 1)
    b.fill([Entry("x", list(range(100, 113)), 0, [12]), Entry("y", [7], 0, [])], s.cache)
    before = {k: b.h[k].copy() for k in ("input_ids", "positions", "slot_mapping0", "block_table0")}
    assert (b.num_tokens, b.num_reqs, b.num_rows, b.max_q_len, b.num_singles) == (14, 2, 1, 13, 1)
    b.pad(4, 32, 4)
    h = b.h
    assert (b.num_tokens, b.num_reqs, b.num_rows, b.max_q_len, b.num_singles) == (32, 4, 4, 17, 2)
    assert b.q_lens == [13, 1, 1, 17] and h["cu_seqlens"][:5].tolist() == [0, 13, 14, 15, 32]
    assert h["seq_lens"][:4].tolist() == [13, 1, 1, 17] and h["state_slots"][2:4].tolist() == [8, 8]
    assert h["positions"][14:32].tolist() == [0] + list(range(17)) and (h["slot_mapping0"][14:32] == -1).all()
    assert h["block_table0"][2:4].tolist() == [[0] * 4] * 2 and h["logits_rows"][:4].tolist() == [12, 14, 14, 14]
    assert (h["feedback_src"][14:32] == -1).all()
    for k, v in before.items():
        assert (b.h[k][:14] == v[:14]).all() if k != "block_table0" else (b.h[k][:2] == v[:2]).all()
    b.pad(4, 32, 4)                                        # nothing to add: nothing changes
    assert (b.num_tokens, b.num_reqs, b.num_rows) == (32, 4, 4)
    for reqs, tokens, rows, needle in ((3, 32, 4, "never cut"), (4, 33, 4, "need a request"), (6, 33, 4, "at least one token"),
                                       (9, 64, 4, "never cut"), (4, 32, 9, "never cut")):
        with pytest.raises(ValueError, match=needle):
            b.pad(reqs, tokens, rows)
    b.fill([Entry("x", list(range(100, 113)), 0, [])], s.cache)   # a step that wants no logits pads none
    b.pad(2, 32, 0)
    assert (b.num_tokens, b.num_reqs, b.num_rows) == (32, 2, 0) and b.q_lens == [13, 19]


def test_limits_are_refused():
    import pytest
    s, b = setup(1000)
    s.cache.admit("x")
    s.cache.allocate("x", 0, 40)
    with pytest.raises(ValueError, match="outside its"):
        b.fill([Entry("x", [1, 2], 0, [2])], s.cache)
    with pytest.raises(ValueError, match="brings no token"):
        b.fill([Entry("x", [1], 0, []), Entry("x", [], 1, [])], s.cache)
    small = StepBatch(torch.device("cpu"), 8, 1, 2, [1])
    with pytest.raises(ValueError, match="tokens in one step"):
        small.fill([Entry("x", list(range(9)), 0, [])], s.cache)
    with pytest.raises(ValueError, match="block table"):
        small.fill([Entry("x", list(range(8)), 0, [])], s.cache)


def test_engine_loop_with_a_stand_in_runner():
    """Engine.generate over scheduler and sampler seams, with a runner that returns one-hot logits
    for token (seq_len % vocab): checks ordering of outputs, chunking, finishing and freeing."""
    from dinfer_amd.engine.engine import Engine

    class FakeModel:
        class spec:
            vocab_size = 50
            eos_token_ids = (49,)

    class FakeRunner:
        def __init__(self):
            self.options = EngineOptions(max_num_seqs=3, max_num_batched_tokens=16, block_size=4, max_model_len=64,
                                         num_blocks=32)
            self.cache = CacheManager([GroupSpec(4, 32)], 3)
            self.model, self.device, self.max_rows, self.steps = FakeModel, torch.device("cpu"), 3, []

        def step_planned(self, scheduler, plan, greedy=False):
            self.steps.append([(x.request.id, x.num_new, x.start) for x in plan.scheduled])
            rows = [(x.start + x.num_new) % 50 for x in plan.scheduled if x.samples]
            return torch.nn.functional.one_hot(torch.tensor(rows, dtype=torch.long), 50).float()

    class FakeSampler:
        def sample(self, logits, rows):
            return logits.argmax(-1).tolist()

        def forget(self, key):
            self.forgotten.append(key)

        forgotten: list = []

    eng = Engine(runner=FakeRunner())
    eng.sampler = FakeSampler()
    outs = eng.generate([list(range(10)), list(range(30)), [1, 2]], SamplingParams(max_tokens=3, temperature=0.0))
    assert outs == [[10, 11, 12], [30, 31, 32], [2, 3, 4]]
    assert sorted(eng.sampler.forgotten) == [0, 1, 2]                          # told of every request that ended
    assert eng.runner.steps[0] == [(0, 10, 0), (1, 6, 0)]                   # budget 16: the second prompt is cut
    assert eng.runner.steps[1] == [(0, 1, 10), (1, 16, 6)]                  # the decode row is exempt: the prompt gets all 16
    assert eng.runner.cache.num_free() == 32 and not eng.has_unfinished()
    outs = eng.generate([[5] * 47], SamplingParams(max_tokens=10, temperature=0.0))
    assert outs == [[47, 48, 49]]                                           # 49 is eos
    st = eng.stats()                                                        # the counters of both runs
    assert (st["prompt_tokens_total"], st["generation_tokens_total"]) == (42 + 47, 9 + 3)
    assert (st["request_success_length"], st["request_success_stop"], st["request_abort"]) == (3, 1, 0)
    assert st["engine_steps_total"] == len(eng.runner.steps) and st["num_preemptions_total"] == 0
    assert (st["num_requests_running"], st["num_requests_waiting"], st["kv_cache_usage"]) == (0, 0, 0.0)
    eng.add_request([1, 2, 3], SamplingParams(max_tokens=5))
    eng.add_request(list(range(20)), SamplingParams(max_tokens=5), request_id="b")
    eng.step()
    st = eng.stats()
    assert st["num_requests_running"] + st["num_requests_waiting"] == 2 and st["kv_cache_usage"] > 0
    eng.abort("b")
    assert eng.stats()["request_abort"] == 1


def test_planned_fill_writes_what_the_entries_would():
    """The scheduler's plan written straight from the core's tokens equals the same step given as entries."""
    import numpy as np
    opt = EngineOptions(max_num_seqs=4, max_num_batched_tokens=12, block_size=4, max_model_len=64, num_blocks=40)
    cache = CacheManager([GroupSpec(4, 40), GroupSpec(4, 40, 6)], 4)
    s = Scheduler(opt, cache, eos_token_ids=[])
    mk = lambda: StepBatch(torch.device("cpu"), 16, 4, 4, [16, 16])
    a, b = mk(), mk()
    for i, n in enumerate((9, 3, 14)):
        s.add_request(Request(i, [100 * i + j for j in range(n)], SamplingParams(max_tokens=4)))
    for step in range(8):
        out = s.schedule()
        if not len(out):
            break
        a.fill_planned(s)
        entries = [Entry(x.request.id, x.request.tokens(x.start, x.num_new), x.start, [x.num_new - 1] if x.samples else [])
                   for x in out.scheduled]
        b.fill(entries, cache)
        assert (a.num_tokens, a.num_reqs, a.num_rows, a.max_q_len, a.max_seq_len, a.num_singles, a.req_ids) == \
               (b.num_tokens, b.num_reqs, b.num_rows, b.max_q_len, b.max_seq_len, b.num_singles, b.req_ids)
        T, B, R = a.num_tokens, a.num_reqs, a.num_rows
        for name, n in (("input_ids", T), ("positions", T), ("slot_mapping0", T), ("slot_mapping1", T),
                        ("cu_seqlens", B + 1), ("seq_lens", B), ("state_slots", B), ("logits_rows", R),
                        ("block_table0", B), ("block_table1", B)):
            assert np.array_equal(a.h[name][:n], b.h[name][:n]), (step, name)
        s.update(out, [7000 + step] * len(out.sampling_requests()))
        cache.check()
    assert step >= 5


def test_rows_of_prompt_positions_follow_the_sampling_rows():
    """A request that wants logits at every prompt position: those rows come after the rows of all requests that
    sample, so the sampler's rows stay the first ones."""
    opt = EngineOptions(max_num_seqs=4, max_num_batched_tokens=64, block_size=16, max_model_len=4096, num_blocks=64,
                        max_logits_rows=10, decode_exempt_from_budget=False)
    cache = CacheManager([GroupSpec(16, 64)], 4)
    s, b = Scheduler(opt, cache, eos_token_ids=[]), StepBatch(torch.device("cpu"), 256, 4, 10, [8])
    s.add_request(Request(1, list(range(100, 104)), SamplingParams(max_tokens=4, prompt_logprobs=0)))
    s.add_request(Request(2, list(range(200, 207)), SamplingParams(max_tokens=4)))
    s.add_request(Request(3, list(range(300, 320)), SamplingParams(max_tokens=4, prompt_logprobs=3)))
    out = s.schedule()
    b.fill_planned(s)
    # request 1: rows at 0..2 and the sampling row 3; request 2 samples at its 7th token; request 3 gets the three
    # rows that are left and is cut there
    assert [(x.request.id, x.num_new, x.samples) for x in out.scheduled] == [(1, 4, True), (2, 7, True), (3, 3, False)]
    assert b.num_rows == 8 and b.h["logits_rows"][:8].tolist() == [3, 10, 0, 1, 2, 11, 12, 13]
    assert [(r.id, p) for r, p in out.prompt_rows()] == [(1, 0), (1, 1), (1, 2), (3, 0), (3, 1), (3, 2)]
    s.update(out, {1: 5, 2: 5})
    out = s.schedule()
    b.fill_planned(s)
    assert [(x.request.id, x.start, x.num_new) for x in out.scheduled] == [(1, 4, 1), (2, 7, 1), (3, 3, 6)]
    assert b.h["logits_rows"][:8].tolist() == [0, 1, 2, 3, 4, 5, 6, 7]
