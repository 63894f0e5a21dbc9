"""Generation through the Python entry point: greedy against the plain implementation on the small workloads
(three prompts of 5/17/33 tokens decoded greedily; four of 1/9/40/70 prefilled in portions of 16 beside decoding
requests and sampled at temperature 0.7), sampling rules through the whole engine, preemption."""
import random

import pytest

import plain_qwen3 as plain
from tiny_configs import CONFIGS, PAGE

pytestmark = pytest.mark.gpu


def engine(model_dir, name, dtype="float32", **kw):
    from dinfer_amd import Engine
    opts = dict(dtype=dtype, max_model_len=CONFIGS[name][0]["max_position_embeddings"], max_num_seqs=4,
                max_num_batched_tokens=64, block_size=PAGE[name], num_blocks=128)
    opts.update(kw)
    return Engine(str(model_dir), **opts)


def prompts_for(name, lens, seed):
    rng = random.Random(seed)
    V = CONFIGS[name][0]["vocab_size"]
    return [[rng.randrange(V) for _ in range(n)] for n in lens]


def plain_greedy(cfg, w, prompt, n):
    """(tokens, margins): greedy continuation by the plain model, with the gap between the two best logits."""
    ids, margins = list(prompt), []
    for _ in range(n):
        row = plain.forward(cfg, w, ids)[-1]
        top = row.topk(2).values
        margins.append(float(top[0] - top[1]))
        ids.append(int(row.argmax()))
    return ids[len(prompt):], margins


@pytest.mark.parametrize("name,lens", [("A", [5, 17, 33]), ("B", [1, 9, 40, 70]), ("C", [3, 50])])
def test_greedy_generation_equals_plain(model_dirs, name, lens):
    """Tiny A's workload (3 prompts of 5/17/33, 8 greedy tokens) and its like on B and C, in 32-bit,
    with a budget that cuts prompts into portions beside decoding requests."""
    from dinfer_amd import SamplingParams
    cfg, w = plain.load(model_dirs[name])
    prompts = prompts_for(name, lens, 7)
    eng = engine(model_dirs[name], name, max_num_batched_tokens=16)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True))
    for p, g in zip(prompts, got):
        want, margins = plain_greedy(cfg, w, p, 8)
        for i, (a, b, m) in enumerate(zip(g, want, margins)):
            assert a == b or m < 1e-4, f"{name}: prompt of {len(p)}, token {i}: {a} != {b} (margin {m})"
            if a != b:
                break
    assert eng.runner.cache.num_free(0) == 128
    eng.runner.cache.check()


def judge_greedy(cfg, w, prompt, tokens, slack=0.1):
    """Every generated token against the plain model's logits after the tokens generated before it: it must be the
    plain model's best, or lie within `slack` of the row's spread below it (bfloat16 logits are off by up to 0.05 of
    the spread each, so two logits nearer than that may change places). Returns how many were the best."""
    ids, best = list(prompt), 0
    for i, tok in enumerate(tokens):
        row = plain.forward(cfg, w, ids)[-1]
        short = float((row.max() - row[tok]) / row.std())
        assert short < slack, f"prompt of {len(prompt)}, output {i}: token {tok} lies {short:.3f} row-sigmas below the best"
        best += short == 0.0
        ids.append(tok)
    return best


@pytest.mark.parametrize("fast", [True, False], ids=["graphs_and_steps_ahead", "eager_step_by_step"])
def test_bfloat16_generation_follows_plain_up_to_near_ties(model_dirs, fast):
    """fast: as the engine serves by default: decode steps replayed from graphs that find their best tokens
    themselves, each launched before the tokens of the one before it are read (its input stays on the device).
    Every token is judged against the plain model's logits after the tokens before it."""
    from dinfer_amd import SamplingParams
    name = "B"
    cfg, w = plain.load(model_dirs[name])
    prompts = prompts_for(name, [9, 40, 70], 8)
    eng = engine(model_dirs[name], name, dtype="bfloat16", hip_graph=fast, async_scheduling=fast)
    got = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert bool(eng.runner._graphs) == fast and (eng.steps_launched_ahead >= 8) == fast
    if fast:
        assert all(greedy for _, greedy in eng.runner._graphs), "the graphs' own argmax chose the tokens"
    best = sum(judge_greedy(cfg, w, p, g) for p, g in zip(prompts, got))
    assert best >= 30, f"only {best} of 36 tokens are the plain model's first choice"


def test_temperature_sampling_with_seed_in_mixed_batches(model_dirs):
    """Tiny B's workload: prompts of 1/9/40/70 prefilled in portions of 16 beside decoding requests,
    12 tokens each at temperature 0.7 with a fixed seed. Every sampled token must be the one the plain
    rule picks from the plain model's logits for (seed, number of outputs so far); and the same
    request gives the same tokens alone as in the batch."""
    from dinfer_amd import SamplingParams
    name = "B"
    cfg, w = plain.load(model_dirs[name])
    prompts = prompts_for(name, [1, 9, 40, 70], 9)
    sps = [SamplingParams(max_tokens=12, temperature=0.7, seed=1000 + i, ignore_eos=True) for i in range(4)]
    eng = engine(model_dirs[name], name, max_num_batched_tokens=16)
    got = eng.generate(prompts, sps)
    judged = 0
    for p, g, sp in zip(prompts, got, sps):
        ids = list(p)
        for i, tok in enumerate(g):
            row = plain.forward(cfg, w, ids)[-1]
            want, slack = plain.sample_row(row, 0.7, sp.seed, i)
            if slack > 2e-5:   # 32-bit logits and sums: anything nearer to an interval's edge may fall either way
                judged += 1
                assert tok == want, f"prompt {len(p)}, output {i}: engine {tok}, rule {want}"
            ids.append(tok)
    assert judged >= 44
    alone = engine(model_dirs[name], name).generate([prompts[2]], sps[2])
    assert alone[0] == got[2]


def test_stop_rules_through_the_engine(model_dirs):
    from dinfer_amd import SamplingParams
    name = "A"
    cfg, w = plain.load(model_dirs[name])
    p = prompts_for(name, [12], 3)[0]
    want, _ = plain_greedy(cfg, w, p, 8)
    eng = engine(model_dirs[name], name)
    stop = want[3]
    got = eng.generate([p], SamplingParams(max_tokens=8, temperature=0.0, stop_token_ids=[stop], ignore_eos=True))[0]
    assert got == want[:want.index(stop) + 1]          # ends with the first occurrence of the stop id
    assert eng.generate([p], SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True))[0] == want[:3]
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([5, 999], SamplingParams())
    with pytest.raises(ValueError, match="top_p"):
        eng.add_request([5], SamplingParams(top_p=0.0))


def test_preemption_recomputes_and_gives_the_same_tokens(model_dirs):
    """A pool too small for all requests: the last running one is preempted, later recomputes its prompt
    and outputs, and still produces the tokens it would have produced alone."""
    from dinfer_amd import SamplingParams
    name = "B"
    prompts = prompts_for(name, [30, 30, 30], 5)
    sp = SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True)
    roomy = engine(model_dirs[name], name).generate(prompts, sp)
    tight = engine(model_dirs[name], name, num_blocks=15, max_model_len=64)   # 15 pages of 8: 120 tokens for 150
    got = tight.generate(prompts, sp)
    assert got == roomy
    assert tight.runner.cache.num_free(0) == 15
    st = tight.stats()
    assert st["num_preemptions_total"] >= 1 and st["prompt_tokens_total"] > 90 and st["generation_tokens_total"] == 60
    assert st["request_success_length"] == 3
    tight.runner.cache.check()


def test_penalties_and_truncation_through_the_engine(model_dirs):
    from dinfer_amd import SamplingParams
    name = "A"
    cfg, w = plain.load(model_dirs[name])
    p = prompts_for(name, [10], 4)[0]
    eng = engine(model_dirs[name], name)
    sp = SamplingParams(max_tokens=6, temperature=0.0, repetition_penalty=1.8, frequency_penalty=0.7, presence_penalty=0.4,
                        ignore_eos=True)
    got = eng.generate([p], sp)[0]
    ids, out = list(p), []
    for _ in range(6):
        row = plain.apply_penalties(plain.forward(cfg, w, ids)[-1], p, out, 1.8, 0.7, 0.4)
        top = row.topk(2).values
        tok = int(row.argmax())
        if float(top[0] - top[1]) < 1e-4:
            break
        out.append(tok)
        ids.append(tok)
    assert got[:len(out)] == out and len(out) >= 3
    sp = SamplingParams(max_tokens=30, temperature=1.5, top_k=3, seed=5, ignore_eos=True)
    got = eng.generate([p], sp)[0]
    ids = list(p)
    seen = set()
    for i, tok in enumerate(got):
        row = plain.forward(cfg, w, ids)[-1]
        best = row.topk(4)
        # one of the best three; the fourth only where it lies within rounding of the third (32-bit logits against
        # the plain model's float64: 1e-4 of the row's spread is a hundred times the engine's error)
        tie = float(best.values[2] - best.values[3]) < 1e-4 * float(row.std())
        assert tok in best.indices[:4 if tie else 3].tolist(), f"output {i}: token {tok} is not among the best three"
        # and the very token the plain rule draws from those three with this seed, where the draw is clear of an edge
        want, slack = plain.sample_row(row, 1.5, 5, i, top_k=3)
        if slack > 1e-3 and not tie:
            assert tok == want, f"output {i}: drew {tok}, the plain rule draws {want}"
            seen.add(tok == int(row.argmax()))
        ids.append(tok)
    assert seen == {True, False}, "the draws took the best token sometimes and another sometimes"


def test_command_line_generate(model_dirs, tmp_path):
    """bin/dinfer generate: token ids in, token ids out, equal to the Python entry point."""
    import json
    import subprocess
    import sys
    from pathlib import Path
    from dinfer_amd import SamplingParams
    root = Path(__file__).resolve().parent.parent
    name = "A"
    prompts = prompts_for(name, [6, 11], 12)
    f = tmp_path / "prompts.jsonl"
    f.write_text(json.dumps(prompts[1]) + "\n")
    p = subprocess.run([sys.executable, str(root / "bin" / "dinfer"), "generate", "--model", str(model_dirs[name]),
                        "--dtype", "float32", "--max-model-len", "128", "--max-num-seqs", "4", "--block-size", "4",
                        "--num-blocks", "64", "--max-num-batched-tokens", "32", "--prompt-ids",
                        ",".join(map(str, prompts[0])), "--prompts-file", str(f), "--max-tokens", "5", "--temperature", "0",
                        "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    got = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")]
    want = engine(model_dirs[name], name).generate(prompts, SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    assert [g["prompt_ids"] for g in got] == prompts and [g["output_ids"] for g in got] == want
    assert all(g["finish_reason"] == "length" and "logprobs" not in g for g in got)
    forced = want[0][0] + 1
    p = subprocess.run([sys.executable, str(root / "bin" / "dinfer"), "generate", "--model", str(model_dirs[name]),
                        "--dtype", "float32", "--max-model-len", "128", "--max-num-seqs", "4", "--block-size", "4",
                        "--num-blocks", "64", "--prompt-ids", ",".join(map(str, prompts[0])), "--max-tokens", "2",
                        "--temperature", "0", "--ignore-eos", "--logprobs", "2", "--prompt-logprobs", "0", "--logit-bias",
                        f"{forced}:100"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    g = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")][0]
    assert g["output_ids"] == [forced] * 2 and [x["token_id"] for x in g["logprobs"]] == [forced] * 2
    assert g["logprobs"][0]["top"][0][0] == want[0][0] and g["logprobs"][0]["rank"] >= 1
    assert g["prompt_logprobs"][0] is None and [x["token_id"] for x in g["prompt_logprobs"][1:]] == prompts[0][1:]
    p = subprocess.run([sys.executable, str(root / "bin" / "dinfer"), "device-info"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0 and "gfx950" in json.loads(p.stdout)["arch"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefix_caching_changes_nothing_but_the_work(model_dirs, dtype):
    """Prompts that share their first 40 tokens, one after the other and then together: with the prefix
    cache the later ones find pages of the earlier ones and compute only their own tail; the tokens
    generated are those of an engine without it (the cached keys and values are the same numbers:
    they depend on the tokens before them only)."""
    from dinfer_amd import SamplingParams
    name = "B"
    stem = prompts_for(name, [40], 21)[0]
    tails = prompts_for(name, [3, 11, 1, 25], 22)
    prompts = [stem + t for t in tails]
    sp = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    plain_eng = engine(model_dirs[name], name, dtype=dtype, enable_prefix_caching=False)
    assert not plain_eng.runner.cache.prefix_caching
    want = [plain_eng.generate([p], sp)[0] for p in prompts] + plain_eng.generate(prompts, sp)
    eng = engine(model_dirs[name], name, dtype=dtype, enable_prefix_caching=True)
    got, cached = [], []
    for p in prompts:                       # one after the other: each finds the stem of the one before
        rid = eng.add_request(p, sp)
        req = eng.scheduler.requests[rid]
        toks = []
        while eng.has_unfinished():
            toks += [o.token for o in eng.step() if o.token is not None]
        got.append(toks)
        cached.append(req.num_cached_tokens)
    page = PAGE[name]
    assert cached[0] == 0 and all(c == 40 // page * page for c in cached[1:]), cached
    assert eng.stats()["prefix_cache_hit_tokens_total"] == sum(cached)
    assert eng.stats()["prompt_tokens_total"] == sum(len(p) for p in prompts) - sum(cached)
    got += eng.generate(prompts, sp)        # all together: pages shared between live requests
    if dtype == "float32":
        assert got == want
    else:
        # bfloat16: a cached page was written by another kernel shape than the one that would write it now, so two
        # nearly equal logits may change places; every token is judged against the plain model instead
        cfg, w = plain.load(model_dirs[name])
        for p, g in zip(prompts + prompts, got):
            judge_greedy(cfg, w, p, g)
    eng.runner.cache.check()
    assert eng.runner.cache.num_free(0) == 128


def test_prefix_cache_is_on_where_every_layer_keeps_its_keys(model_dirs):
    """Left to itself the engine reuses pages between requests, except for a model with window layers (their
    pages go back while the request lives); asking for it there is an error, not a silent no."""
    assert engine(model_dirs["A"], "A").runner.cache.prefix_caching
    assert not engine(model_dirs["C"], "C").runner.cache.prefix_caching
    assert not engine(model_dirs["A"], "A", enable_prefix_caching=False).runner.cache.prefix_caching
    with pytest.raises(ValueError, match="keep every key"):
        engine(model_dirs["C"], "C", enable_prefix_caching=True)


@pytest.mark.parametrize("seed", range(12))
def test_random_workloads_equal_the_plain_continuations(seed, tmp_path):
    """Requests that arrive over time, share prompt stems (the prefix cache is on where the model allows), are cut
    by small budgets, meet a pool so small that some are preempted, and are aborted now and then; graphs on or off.
    In 32-bit, every request that finishes has generated exactly the plain implementation's greedy continuation,
    and every page is back at the end. Some requests ask for the log-probabilities of their outputs or of their
    prompts (with few rows to spare, so those prompts come in small portions): each value against the plain
    log-softmax, every prompt position once and in order, and nobody's tokens change."""
    from dinfer_amd import Engine, SamplingParams
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.weights import write_random_model
    rng, rng2 = random.Random(500 + seed), random.Random(900 + seed)
    name = "ABC"[seed % 3]
    cfgd, page = CONFIGS[name][0], PAGE[name]
    write_random_model(Qwen3Config.from_dict(cfgd), tmp_path, seed=seed, dtype="float32")
    cfg, w = plain.load(tmp_path)
    nblocks = rng.choice([12, 20, 40])
    maxlen = min(cfgd["max_position_embeddings"], nblocks * page)
    seqs = rng.choice([2, 4])
    eng = Engine(str(tmp_path), dtype="float32", max_model_len=maxlen, max_num_seqs=seqs,
                 max_num_batched_tokens=rng.choice([8, 16, 64]), block_size=page, num_blocks=nblocks,
                 hip_graph=seed % 2 == 0, max_logits_rows=seqs + rng2.choice([1, 3, 8]))
    V = cfgd["vocab_size"]
    stems = [[rng.randrange(V) for _ in range(rng.randint(1, 3 * page))] for _ in range(2)]
    arrivals = []
    for _ in range(rng.randint(4, 8)):
        p = (rng.choice(stems) if rng.random() < 0.6 else []) + [rng.randrange(V) for _ in range(rng.randint(1, 2 * page))]
        n = rng.randint(1, 8)
        arrivals.append((rng.randint(0, 12), p[:maxlen - n], n))
    arrivals.sort(key=lambda x: x[0])
    asked, got, aborted, step = {}, {}, set(), 0
    about, about_prompt, options = {}, {}, {}
    while arrivals or eng.has_unfinished():
        while arrivals and arrivals[0][0] <= step:
            _, p, n = arrivals.pop(0)
            sp = SamplingParams(max_tokens=n, temperature=0.0, ignore_eos=True,
                                logprobs=rng2.choice([None, None, 0, 2]), prompt_logprobs=rng2.choice([None, None, 0, 1]))
            rid = eng.add_request(p, sp)
            asked[rid], got[rid], about[rid], about_prompt[rid], options[rid] = (p, n), [], [], [], sp
        if rng.random() < 0.04 and got:
            victim = rng.choice(list(got))
            if len(got[victim]) < asked[victim][1]:
                eng.abort(victim)
                aborted.add(victim)
        for o in eng.step():
            if o.token is not None:
                got[o.request_id].append(o.token)
                about[o.request_id].append(o.logprobs)
            about_prompt[o.request_id] += o.prompt_logprobs or []
        step += 1
        assert step < 2000, "the engine makes no progress"
    eng.runner.cache.check()
    assert all(eng.runner.cache.num_free(g) == nblocks for g in range(len(eng.runner.group_specs)))
    for rid, (p, n) in asked.items():
        if rid in aborted:
            continue
        ids, sp = list(p), options[rid]
        for i in range(n):
            row = plain.forward(cfg, w, ids)[-1]
            ids.append(int(row.argmax()))
            if sp.logprobs is not None and len(got[rid]) > i and got[rid][i] == ids[-1]:
                lp = about[rid][i]
                want = plain.token_logprobs(row, ids[-1], 0)[0]
                assert lp.token_id == ids[-1] and abs(lp.logprob - want) < 1e-4 and len(lp.top) == sp.logprobs
        assert got[rid] == ids[len(p):], f"request {rid} (prompt of {len(p)}): {got[rid]} != {ids[len(p):]}"
        if sp.logprobs is None:
            assert about[rid] == [None] * n
        if sp.prompt_logprobs is None:
            assert about_prompt[rid] == []
        else:
            assert [pos for pos, _ in about_prompt[rid]] == list(range(1, len(p)))
            rows = plain.forward(cfg, w, p)
            for pos, lp in about_prompt[rid]:
                want = plain.token_logprobs(rows[pos - 1], p[pos], 0)[0]
                assert lp.token_id == p[pos] and abs(lp.logprob - want) < 1e-4 and len(lp.top) == sp.prompt_logprobs


@pytest.mark.parametrize("dtype,graph", [("float32", False), ("bfloat16", True), ("bfloat16", False)])
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_launched_ahead_give_the_same_tokens(model_dirs, name, dtype, graph):
    """async_scheduling launches a decode step before the tokens of the one before it are read (its input tokens stay
    on the device). Greedy and seeded sampling, ends by length and by a stop token nobody can foresee, requests that
    arrive while others decode: token for token what the engine gives step by step (the same kernels on the same
    inputs: equal, not close)."""
    from dinfer_amd import SamplingParams
    prompts = prompts_for(name, [5, 17, 33, 9, 3, 21], 11)

    def run(ahead, stop=()):
        eng = engine(model_dirs[name], name, dtype=dtype, hip_graph=graph, async_scheduling=ahead, max_num_seqs=4)
        sps = [SamplingParams(max_tokens=n, temperature=t, top_k=k, seed=100 + i, ignore_eos=True, stop_token_ids=list(stop))
               for i, (n, t, k) in enumerate([(24, 0.0, -1), (7, 0.8, -1), (30, 0.0, -1), (13, 1.0, 5), (1, 0.0, -1), (18, 0.7, -1)])]
        ids = [eng.add_request(p, sp) for p, sp in zip(prompts[:4], sps[:4])]
        got, reasons, steps, looked = {}, {}, 0, 0
        while eng.has_unfinished():
            if steps == 9:                       # two more arrive while the first four decode
                ids += [eng.add_request(p, sp) for p, sp in zip(prompts[4:], sps[4:])]
            looked += eng._running is not None   # a step was in flight when this call began
            for o in eng.step():
                if o.token is not None:
                    got.setdefault(o.request_id, []).append(o.token)
                if o.finished:
                    reasons[o.request_id] = o.finish_reason
            steps += 1
            assert steps < 400
        assert eng.runner.cache.num_free(0) == 128
        eng.runner.cache.check()
        return [got[i] for i in ids], [reasons[i] for i in ids], looked

    plain_tokens, plain_reasons, none_ahead = run(False)
    assert none_ahead == 0
    ahead_tokens, ahead_reasons, looked = run(True)
    assert looked > 15, "the decode steps were not launched ahead"
    assert ahead_tokens == plain_tokens and ahead_reasons == plain_reasons
    # a stop token in the middle of the longest output: that request ends while its next step is in flight already
    stop = plain_tokens[2][11]
    a, ra, _ = run(False, stop=[stop])
    b, rb, _ = run(True, stop=[stop])
    assert a == b and ra == rb and "stop" in ra


@pytest.mark.parametrize("ahead", [False, True])
def test_logprobs_and_logit_bias_through_the_engine(model_dirs, ahead):
    """A request that asks for log-probabilities gets, for every token, the plain model's log-softmax at that place
    (of the logits before any bias), also when steps are launched ahead; a bias of +100 makes its token the only
    one that comes, a bias of -100 on the plain model's choice keeps it away."""
    from dinfer_amd import SamplingParams
    name = "B"
    cfg, w = plain.load(model_dirs[name])
    V = cfg["vocab_size"]
    prompts = prompts_for(name, [9, 40, 21, 5], 13)
    first = [int(plain.forward(cfg, w, p)[-1].argmax()) for p in prompts]
    sps = [SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True, logprobs=4),
           SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True, logprobs=0, logit_bias={V - 2: 100.0}),
           SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True, logit_bias={first[2]: -100.0}, logprobs=1),
           SamplingParams(max_tokens=10, temperature=0.8, seed=3, ignore_eos=True)]
    eng = engine(model_dirs[name], name, async_scheduling=ahead, max_num_batched_tokens=32)
    res = eng.generate(prompts, sps, details=True)
    got, about = [g.token_ids for g in res], [g.logprobs for g in res]
    assert [g.finish_reason for g in res] == ["length"] * 4 and all(g.prompt_logprobs is None for g in res)
    assert about[3] is None and got[1] == [V - 2] * 10 and got[2][0] != first[2]
    for p, g, a, sp in zip(prompts[:3], got[:3], about[:3], sps[:3]):
        assert len(a) == len(g)
        ids = list(p)
        for i, (tok, lp) in enumerate(zip(g, a)):
            row = plain.forward(cfg, w, ids)[-1]
            want, rank, top = plain.token_logprobs(row, tok, sp.logprobs)
            assert lp.token_id == tok and abs(lp.logprob - want) < 1e-4, (len(p), i, lp, want)
            gap = float((row.sort(descending=True).values[:-1] - row.sort(descending=True).values[1:])[:sp.logprobs + 1].min())
            if gap > 1e-4:          # (two logits nearer than rounding may change places)
                assert lp.rank == rank and [t for t, _ in lp.top] == [t for t, _ in top], (len(p), i)
            for (_, x), (_, y) in zip(lp.top, top):
                assert abs(x - y) < 1e-4
            ids.append(tok)
    assert all(x.rank == 0 and x.top[0][0] == x.token_id for x in about[0])
    assert eng.runner.cache.num_free(0) == 128


def test_logprobs_in_bfloat16_graphs_equal_step_by_step(model_dirs):
    """Greedy rows whose token a replayed graph finds itself still get their log-probabilities, the same ones
    with and without steps launched ahead."""
    from dinfer_amd import SamplingParams
    prompts = prompts_for("A", [5, 17, 33], 3)
    sp = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True, logprobs=3)
    runs = []
    for ahead in (False, True):
        eng = engine(model_dirs["A"], "A", dtype="bfloat16", hip_graph=True, async_scheduling=ahead)
        runs.append(eng.generate(prompts, sp, details=True))
    assert runs[0] == runs[1]
    assert all(x.rank == 0 and x.top[0] == (x.token_id, x.logprob) for g in runs[0] for x in g.logprobs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_log_probabilities_of_the_prompt(model_dirs, dtype):
    """prompt_logprobs: every token of the prompt but the first, given the tokens before it, against the plain
    model's log-softmax at the position before; prompts longer than the spare rows come in several portions, beside
    requests that decode, and a prompt that is in the prefix cache already is still computed."""
    from dinfer_amd import SamplingParams
    name = "B"
    cfg, w = plain.load(model_dirs[name])
    prompts = prompts_for(name, [40, 9, 70, 2], 17)
    prompts.append(list(prompts[0]))                          # the same prompt again
    sps = [SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True),
           SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True, prompt_logprobs=0),
           SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True, prompt_logprobs=3, logprobs=1),
           SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True, prompt_logprobs=1),
           SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True, prompt_logprobs=2)]
    eng = engine(model_dirs[name], name, dtype=dtype, max_num_batched_tokens=48, max_logits_rows=4 + 20)
    first = eng.generate(prompts[:4], sps[:4], details=True)
    res = first + eng.generate(prompts[4:], sps[4:], details=True)
    assert res[0].prompt_logprobs is None and res[0].logprobs is None and len(res[2].logprobs) == 3
    for p, sp, g in zip(prompts[1:], sps[1:], res[1:]):
        got = g.prompt_logprobs
        assert len(got) == len(p) and got[0] is None
        rows = plain.forward(cfg, w, p)
        for i in range(1, len(p)):
            want, rank, top = plain.token_logprobs(rows[i - 1], p[i], sp.prompt_logprobs)
            # (bfloat16 logits are off by up to 0.05 of the row's spread each, as everywhere in these tests)
            tol = 1e-4 if dtype == "float32" else 0.08 * float(rows[i - 1].std())
            assert got[i].token_id == p[i] and abs(got[i].logprob - want) < tol, (len(p), i, got[i], want)
            assert len(got[i].top) == sp.prompt_logprobs
            if dtype == "float32":
                for (_, x), (_, y) in zip(got[i].top, top):
                    assert abs(x - y) < tol
    assert res[4].token_ids == res[0].token_ids[:3] or dtype != "float32"
    assert eng.runner.cache.num_free(0) == 128
    with pytest.raises(ValueError, match="max_logits_rows"):
        engine(model_dirs[name], name).generate([[1, 2, 3]], SamplingParams(prompt_logprobs=0, max_tokens=1))
