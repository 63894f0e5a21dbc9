"""The engine against the plain implementation: whole prompts, decoding after a prompt,
portions of changing size, mixed batches with reused pages; 32-bit and bfloat16."""
import os
import random

import pytest
import torch

import plain_qwen3 as plain
from tiny_configs import CONFIGS, PAGE

pytestmark = pytest.mark.gpu

# 32-bit path against the float64 plain model: rounding only.
F32_TOL = dict(rtol=2e-4, atol=2e-5)


def make_runner(model_dir, name, dtype, max_tokens=2048, num_blocks=None, max_seqs=4, max_len=None, graph=False):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    cfg = CONFIGS[name][0]
    opt = EngineOptions(dtype=dtype, max_model_len=max_len or cfg["max_position_embeddings"], max_num_seqs=max_seqs,
                        max_num_batched_tokens=max_tokens, block_size=PAGE[name], num_blocks=num_blocks or 256,
                        max_logits_rows=max_tokens, decode_exempt_from_budget=False, hip_graph=graph)
    return ModelRunner.from_dir(model_dir, opt)


def tokens_for(name, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(CONFIGS[name][0]["vocab_size"]) for _ in range(n)]


def check_logits(got, want, dtype, what):
    got = got.double().cpu()
    if dtype == "float32":
        torch.testing.assert_close(got, want, **F32_TOL, msg=lambda m: f"{what}: {m}")
    else:
        # bfloat16 activations: error relative to the spread of the logits of a row
        scale = want.std(dim=-1, keepdim=True)
        err = ((got - want).abs() / scale).max().item()
        rms = ((got - want).pow(2).mean(dim=-1, keepdim=True).sqrt() / scale).max().item()
        if os.environ.get("DINFER_TEST_REPORT"):
            print(f"[report] {what}: max {err:.4f} rms {rms:.4f} row-sigmas", flush=True)
        assert err < 0.08, f"{what}: bf16 logits off by {err:.3f} row-sigmas"
        # the error of a whole row: roundings to 8 bits add up to 0.005 to 0.012 of the row's spread through these
        # models; one key too many or too few in a window of 24, or a gain applied twice, is several times that
        assert rms < 0.02, f"{what}: bf16 logits of a row off by {rms:.4f} row-sigmas (root mean square)"
        gap = want.topk(2, dim=-1).values
        sure = (gap[:, 0] - gap[:, 1]) > 0.25 * scale[:, 0]
        assert (got.argmax(-1)[sure] == want.argmax(-1)[sure]).all(), f"{what}: argmax differs on a clear row"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompt(model_dirs, name, dtype):
    from dinfer_amd.engine.batch import Entry
    cfg, w = plain.load(model_dirs[name])
    r = make_runner(model_dirs[name], name, dtype)
    for n, seed in ((1, 1), (5, 2), (17, 3), (70, 4)):
        ids = tokens_for(name, n, seed)
        want = plain.forward(cfg, w, ids)
        assert r.reserve("x", 0, n)
        got = r.step([Entry("x", ids, 0, list(range(n)))])
        check_logits(got, want, dtype, f"{name} whole prompt of {n}")
        r.finish("x")
    r.cache.check()


# ---- replay helpers ------------------------------------------------------------------------------
def replay(runner, steps):
    """steps: list of (entries, ends); entries: list of (id, tokens, want). Returns {(id, position): row}."""
    from dinfer_amd.engine.batch import Entry
    computed, rows = {}, {}
    for entries, ends in steps:
        es = []
        for rid, toks, want in entries:
            start = computed.get(rid, 0)
            assert runner.reserve(rid, start, len(toks)), f"out of pages for {rid}"
            es.append(Entry(rid, toks, start, want))
        if es:
            logits = runner.step(es).double().cpu()
            i = 0
            for e in es:
                for w in e.want:
                    rows[(e.req_id, e.start + w)] = logits[i]
                    i += 1
                computed[e.req_id] = e.start + len(e.tokens)
                runner.advance(e.req_id, computed[e.req_id])
        for rid in ends:
            runner.finish(rid)
            del computed[rid]
        runner.cache.check()
    return rows


def compare_rows(rows, plain_logits, dtype, what):
    """plain_logits: {id: [T, V]}; every replayed row against the whole-sequence logits."""
    assert rows, "nothing was replayed"
    for rid in {k[0] for k in rows}:
        pos = sorted(p for (r, p) in rows if r == rid)
        got = torch.stack([rows[(rid, p)] for p in pos])
        check_logits(got, plain_logits[rid][pos], dtype, f"{what} request {rid}")


def cut(ids, sizes):
    out, i, k = [], 0, 0
    while i < len(ids):
        n = sizes[k % len(sizes)]
        out.append(ids[i:i + n])
        i += n
        k += 1
    return out


DTYPES = ["float32", "bfloat16"]
NAMES = ["A", "B", "C"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_decode_one_by_one(model_dirs, name, dtype):
    cfg, w = plain.load(model_dirs[name])
    r = make_runner(model_dirs[name], name, dtype)
    ids = tokens_for(name, 100, 5)
    want = {"x": plain.forward(cfg, w, ids)}
    steps = [([("x", ids[:68], [67])], [])]
    steps += [([("x", [ids[p]], [0])], []) for p in range(68, 100)]
    compare_rows(replay(r, steps), want, dtype, f"{name} decode after prompt")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(model_dirs, name, dtype):
    cfg, w = plain.load(model_dirs[name])
    r = make_runner(model_dirs[name], name, dtype)
    ids = tokens_for(name, 117, 6)
    want = {"x": plain.forward(cfg, w, ids)}
    steps = [([("x", part, list(range(len(part))))], []) for part in cut(ids, [7, 16, 2, 5, 3, 33, 2, 8, 1])]
    compare_rows(replay(r, steps), want, dtype, f"{name} portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_requests_with_reused_pages(model_dirs, name, dtype):
    """Up to four live requests, portions of some beside decoded tokens of others; the pool is
    so small that pages of finished requests go to later ones while stale keys still lie in them."""
    cfg, w = plain.load(model_dirs[name])
    page = PAGE[name]
    lens = {"a": 70, "b": 41, "c": 9, "d": 55, "e": 64, "f": 1, "g": 37}
    seqs = {k: tokens_for(name, n, 100 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: plain.forward(cfg, w, v) for k, v in seqs.items()}
    # a, b, c, d start; as each ends the next of e, f, g takes its pages
    pool_tokens = sum(-(-lens[k] // page) * page for k in "abde") + 2 * page
    r = make_runner(model_dirs[name], name, dtype, num_blocks=pool_tokens // page, max_len=128)
    rng = random.Random(9)
    todo = list(seqs)
    live, fed, steps = [], {}, []
    while todo or live:
        while todo and len(live) < 4:
            k = todo.pop(0)
            live.append(k)
            fed[k] = 0
        entries, ends = [], []
        for k in list(live):
            left = lens[k] - fed[k]
            if fed[k] > 0 and left <= 12:
                n = 1  # decode the tail one by one
            elif rng.random() < 0.2 and fed[k] > 0:
                continue  # left out of this step, goes on later
            else:
                n = min(left, rng.choice([2, 3, 5, 8, 13, 16, 21]))
            entries.append((k, seqs[k][fed[k]:fed[k] + n], list(range(n))))
            fed[k] += n
            if fed[k] == lens[k]:
                ends.append(k)
                live.remove(k)
        steps.append((entries, ends))
    rows = replay(r, steps)
    assert len(rows) == sum(lens.values())
    compare_rows(rows, want, dtype, f"{name} mixed")
    assert r.cache.num_free(0) == r.num_blocks


_plain_cache: dict = {}


def plain_logits_of(model_dirs, name, seqs):
    """{id: plain logits [T, V]} of whole sequences (kept: the same sequences serve several parametrisations)."""
    key = (name, tuple((k, tuple(v)) for k, v in sorted(seqs.items(), key=lambda kv: str(kv[0]))))
    if key not in _plain_cache:
        cfg, w = plain.load(model_dirs[name])
        _plain_cache[key] = {k: plain.forward(cfg, w, v) for k, v in seqs.items()}
    return _plain_cache[key]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_many_decoding_requests_beside_prompt_portions(model_dirs, name, dtype):
    """Up to eight live requests: most of them decode (one token a step) while one or two others bring portions
    of their prompts, which is the step a serving engine runs most of the time and which takes its own route
    through the attention kernels (split-K for the single rows, the prompt kernel for the others, in one step).
    The pool holds little more than the eight largest, so pages pass from finished requests to later ones."""
    page = PAGE[name]
    rng = random.Random(31)
    lens = {k: rng.randrange(45, 110) for k in "abcdefghijklmn"}
    prompt = {k: rng.randrange(5, n - 30) for k, n in lens.items()}     # fed in portions; the rest one by one
    seqs = {k: tokens_for(name, n, 500 + i) for i, (k, n) in enumerate(lens.items())}
    want = plain_logits_of(model_dirs, name, seqs)
    pool = sum(sorted(-(-n // page) for n in lens.values())[-8:]) + 2
    r = make_runner(model_dirs[name], name, dtype, num_blocks=pool, max_len=128, max_seqs=8)
    todo, live, fed, steps = list(seqs), [], {}, []
    busy_steps = 0
    while todo or live:
        # one new request every other step, so that prompts arrive while the others are decoding
        if todo and len(live) < 8 and (len(steps) % 2 == 0 or not live):
            k = todo.pop(0)
            live.append(k)
            fed[k] = 0
        entries, ends, singles, portions = [], [], 0, 0
        for k in list(live):
            if fed[k] >= prompt[k]:
                n = 1
                singles += 1
            else:
                n = min(prompt[k] - fed[k], rng.choice([2, 3, 7, 16, 21]))
                portions += n > 1
                singles += n == 1
            entries.append((k, seqs[k][fed[k]:fed[k] + n], list(range(n))))
            fed[k] += n
            if fed[k] == lens[k]:
                ends.append(k)
                live.remove(k)
        busy_steps += singles >= 4 and portions >= 1
        steps.append((entries, ends))
    assert busy_steps >= 10, "the schedule must hold steps with four or more single rows beside a portion"
    rows = replay(r, steps)
    assert len(rows) == sum(lens.values())
    compare_rows(rows, want, dtype, f"{name} many live")
    assert all(r.cache.num_free(g) == r.num_blocks for g in range(len(r.group_specs)))


# (requests, dtype): 33 is padded to a graph of 40 rows, 44 to one of 48; 128 requests at two kv heads are where the
# parts of a request are few enough for the kernel that merges them inside a workgroup
MANY = [(33, "bfloat16"), (44, "bfloat16"), (64, "bfloat16"), (128, "bfloat16"), (64, "float32")]


@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
@pytest.mark.parametrize("num,dtype", MANY)
@pytest.mark.parametrize("name", ["B", "C"])
def test_decoding_with_many_requests(model_dirs, name, num, dtype, graph):
    """33 to 128 requests decode side by side for 40 steps from prompts of unequal length: the row counts at
    which the products, the attention kernels and the graph buckets take other forms than at a handful of rows.
    Every decoded row is compared with the plain model."""
    steps_n = 40
    rng = random.Random(num)
    plen = {i: rng.randrange(1, 60) for i in range(num)}
    seqs = {i: tokens_for(name, plen[i] + steps_n, 900 + i) for i in range(num)}
    want = plain_logits_of(model_dirs, name, seqs)
    r = make_runner(model_dirs[name], name, dtype, max_tokens=1024, num_blocks=num * (-(-100 // PAGE[name])) + 4,
                    max_len=128, max_seqs=num, graph=graph)
    steps, group = [], []
    for i in range(num):                       # prompts, sixteen requests a step
        group.append((i, seqs[i][:plen[i]], [plen[i] - 1]))
        if len(group) == 16 or i == num - 1:
            steps.append((group, []))
            group = []
    for s in range(steps_n - 1):
        steps.append(([(i, [seqs[i][plen[i] + s]], [0]) for i in range(num)], []))
    steps.append(([(i, [seqs[i][plen[i] + steps_n - 1]], [0]) for i in range(num)], list(range(num))))
    rows = replay(r, steps)
    assert bool(r._graphs) == graph
    compare_rows(rows, want, dtype, f"{name} {num} decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(model_dirs, dtype):
    """Three requests decoded side by side for 200 steps from short prompts."""
    name = "C"
    cfg, w = plain.load(model_dirs[name])
    r = make_runner(model_dirs[name], name, dtype, max_len=256)
    seqs = {k: tokens_for(name, 3 + 200 + i, 40 + i) for i, k in enumerate("pqr")}
    want = {k: plain.forward(cfg, w, v) for k, v in seqs.items()}
    steps = [([(k, v[:3 + i], [2 + i]) for i, (k, v) in enumerate(seqs.items())], [])]
    for s in range(200):
        steps.append(([(k, [v[3 + i + s]], [0]) for i, (k, v) in enumerate(seqs.items())], []))
    compare_rows(replay(r, steps), want, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_first_tokens(model_dirs, name, dtype):
    """The first positions of a sequence, fed one token a step from the very first."""
    cfg, w = plain.load(model_dirs[name])
    r = make_runner(model_dirs[name], name, dtype)
    ids = tokens_for(name, 6, 77)
    want = {"x": plain.forward(cfg, w, ids)}
    steps = [([("x", [t], [0])], []) for t in ids]
    compare_rows(replay(r, steps), want, dtype, f"{name} first tokens")


def test_modes_agree_closely_in_32bit(model_dirs):
    """In 32-bit every row's arithmetic is fixed by its own position: whole, token by token and
    chunked replays give the same logits to the last bits (not merely within the plain tolerance)."""
    name = "B"
    r = make_runner(model_dirs[name], name, "float32")
    ids = tokens_for(name, 60, 8)
    whole = replay(r, [([("x", ids, list(range(60)))], ["x"])])
    single = replay(r, [([("y", [t], [0])], []) for t in ids])
    parts = replay(r, [([("z", p, list(range(len(p))))], []) for p in cut(ids, [7, 2, 16, 5])])
    for p in range(60):
        assert torch.equal(whole[("x", p)], single[("y", p)]), f"position {p}: token-by-token differs"
        assert torch.equal(whole[("x", p)], parts[("z", p)]), f"position {p}: portions differ"


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_graph_replays_equal_eager(model_dirs, dtype):
    """Decode steps replayed from a captured HIP graph against the same steps run eagerly: every
    replay is checked, with eager work (prompt portions of other requests) between the replays,
    and with batches that grow and shrink across the graph's size buckets."""
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    name = "B"
    cfg = CONFIGS[name][0]
    seqs = {k: tokens_for(name, 60 + 7 * i, 300 + i) for i, k in enumerate("abc")}
    runners = {}
    for graph in (False, True):
        opt = EngineOptions(dtype=dtype, max_model_len=cfg["max_position_embeddings"], max_num_seqs=4,
                            max_num_batched_tokens=64, block_size=PAGE[name], num_blocks=128, max_logits_rows=64,
                            decode_exempt_from_budget=False, hip_graph=graph)
        runners[graph] = ModelRunner.from_dir(model_dirs[name], opt)
    steps = [([("a", seqs["a"][:20], [19])], [])]
    steps += [([("a", [seqs["a"][20 + i]], [0])], []) for i in range(3)]                    # bucket 1
    steps += [([("b", seqs["b"][:33], [32])], [])]                                          # eager in between
    steps += [([("a", [seqs["a"][23 + i]], [0]), ("b", [seqs["b"][33 + i]], [0])], []) for i in range(4)]  # bucket 2
    steps += [([("c", seqs["c"][:9], [])], [])]
    steps += [([(k, [seqs[k][n + i]], [0]) for k, n in (("a", 27), ("b", 37), ("c", 9))], []) for i in range(5)]  # bucket 4
    steps += [([("b", [seqs["b"][42]], [0])], ["a"])]                                       # back to bucket 1
    eager, replayed = replay(runners[False], steps), replay(runners[True], steps)
    assert runners[True]._graphs and not runners[False]._graphs
    assert eager.keys() == replayed.keys()
    for k in eager:
        # same kernels; only the split of the keys differs (the graph splits for the longest possible request)
        torch.testing.assert_close(replayed[k], eager[k], rtol=1e-3, atol=1e-3, msg=lambda m: f"{k}: {m}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_steps_with_portions_replayed_from_graphs(model_dirs, name, dtype):
    """A serving schedule: one request at a time brings its prompt in portions of 16 while up to four others decode,
    each wanting one row at most. Steps whose counts (tokens, requests, longest portion) come up again are padded with
    made-up requests and replayed from a graph captured the second time. Every wanted row against the plain model, and
    against the same schedule run eagerly without padding: in 32-bit bit for bit (a row's arithmetic is its own), in
    bfloat16 closely (a padded step of 17 to 32 rows does not take the norms along in its products where the unpadded
    step of up to 16 rows does)."""
    rng = random.Random(17)
    ids = "abcdefghij"
    plen = {k: rng.randrange(20, 75) for k in ids}
    outs = {k: rng.randrange(6, 14) for k in ids}
    seqs = {k: tokens_for(name, plen[k] + outs[k], 700 + i) for i, k in enumerate(ids)}
    want = plain_logits_of(model_dirs, name, seqs)
    todo, live, fed, steps = list(ids), [], {}, []
    while todo or live:
        filling = [k for k in live if fed[k] < plen[k]]
        if todo and len(live) < 5 and not filling:
            k = todo.pop(0)
            live.append(k)
            fed[k] = 0
        entries, ends = [], []
        for k in list(live):
            n = min(16, plen[k] - fed[k]) if fed[k] < plen[k] else 1
            last = fed[k] + n >= plen[k]                    # the row after the prompt's last token, then every row
            entries.append((k, seqs[k][fed[k]:fed[k] + n], [n - 1] if last else []))
            fed[k] += n
            if fed[k] == len(seqs[k]):
                ends.append(k)
                live.remove(k)
        steps.append((entries, ends))
    page = PAGE[name]
    got = {}
    for graph in (False, True):
        r = make_runner(model_dirs[name], name, dtype, max_tokens=64, max_len=128, max_seqs=8, graph=graph,
                        num_blocks=8 * (-(-128 // page)) + 2)
        got[graph] = replay(r, steps)
        assert all(r.cache.num_free(g) == r.num_blocks for g in range(len(r.group_specs)))
        if graph:
            assert len(r._portion_graphs) >= 3 and r.portion_replays >= 10, (len(r._portion_graphs), r.portion_replays)
        else:
            assert not r._portion_graphs and r.portion_replays == 0
    compare_rows(got[True], want, dtype, f"{name} portions from graphs")
    assert got[True].keys() == got[False].keys()
    for k in got[True]:
        if dtype == "float32":
            assert torch.equal(got[True][k], got[False][k]), f"{k}: the replayed step differs from the eager one"
        else:
            spread = got[False][k].std()
            assert float((got[True][k] - got[False][k]).abs().max() / spread) < 0.08, k
