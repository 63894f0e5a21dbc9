"""Two layers with the layer sizes of Qwen3-8B, 14B and 32B (group sizes 4, 5 and 8; H * D equal to, and larger
than, the hidden size), random weights, against the plain implementation in 32-bit and in bfloat16: whole prompt,
decoding, a second request beside it; then the steps a loaded engine runs: eight live requests with most of them
decoding beside prompt portions, and 40 and 64 requests decoding, eagerly and from captured graphs. The vocabulary
is cut to 2048 rows, which is no layer size. The plain model runs in float64 with torch's own operations, here on
the GPU (on the CPU these sizes take minutes)."""
import os
import random

import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu

SHAPES = {
    "8B": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, intermediate_size=12288),
    "14B": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=17408),
    "32B": dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, intermediate_size=25600),
}
VOCAB = 2048


@pytest.fixture(scope="module")
def big_models(tmp_path_factory):
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.weights import write_random_model
    out = {}
    for name, sizes in SHAPES.items():
        cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=VOCAB, head_dim=128, num_hidden_layers=2,
                   rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=512, tie_word_embeddings=False, **sizes)
        d = tmp_path_factory.mktemp(f"big_{name}")
        write_random_model(Qwen3Config.from_dict(cfg), d, seed=len(name))
        out[name] = d
    return out


class PlainOnGpu:
    """The plain model of one folder with float64 weights on the GPU; logits come back on the CPU."""

    def __init__(self, model_dir):
        self.cfg, w = plain.load(model_dir, dtype=torch.float32)
        self.w = {k: v.cuda().double() for k, v in w.items()}
        self.done = {}

    def forward(self, ids):
        key = tuple(ids)
        if key not in self.done:
            with torch.device("cuda"):
                self.done[key] = plain.forward(self.cfg, self.w, ids).cpu()
        return self.done[key]


@pytest.fixture(scope="module")
def plain_models(big_models):
    """One plain model at a time (float64 weights of these sizes are 3 to 8 GB)."""
    held = {}

    def get(name):
        if name not in held:
            held.clear()
            torch.cuda.empty_cache()
            held[name] = PlainOnGpu(big_models[name])
        return held[name]

    yield get
    held.clear()
    torch.cuda.empty_cache()


def tokens(n, seed):
    rng = random.Random(seed)
    return [rng.randrange(VOCAB) for _ in range(n)]


def check(got, ref, dtype, what):
    got = got.double()
    spread = ref.std(-1, keepdim=True)
    if os.environ.get("DINFER_TEST_REPORT"):
        print(f"[report] {dtype} {what}: max {((got - ref).abs() / spread).max().item():.3e} rms "
              f"{((got - ref).pow(2).mean(-1, keepdim=True).sqrt() / spread).max().item():.3e}", flush=True)
    if dtype == "float32":
        # float sums of up to 25,600 terms in a fixed order against float64: an error of a few 1e-6 of the row's spread
        # for each of the dozen products between the tokens and the logits
        err = ((got - ref).abs() / spread).max().item()
        assert err < 1e-4, f"{what}: 32-bit logits off by {err:.2e} of the row's spread"
    else:
        err = ((got - ref).abs() / spread).max().item()
        rms = ((got - ref).pow(2).mean(-1, keepdim=True).sqrt() / spread).max().item()
        assert err < 0.08 and rms < 0.02, f"{what}: bf16 logits off by {err:.3f} (rms {rms:.4f}) row-sigmas"
        top2 = ref.topk(2, -1).values
        clear = (top2[:, 0] - top2[:, 1]) > 0.25 * spread[:, 0]
        assert bool((got.argmax(-1)[clear] == ref.argmax(-1)[clear]).all()), f"{what}: argmax differs on a clear row"


def run_steps(r, steps, want, dtype, what, ends=None):
    """steps: lists of (id, tokens, want); every wanted row against the plain logits of its sequence.
    ends: {step index: ids that are finished after that step}."""
    from dinfer_amd.engine.batch import Entry
    fed = {}
    for n, st in enumerate(steps):
        entries = []
        for rid, toks, wants in st:
            start = fed.get(rid, 0)
            assert r.reserve(rid, start, len(toks))
            entries.append(Entry(rid, toks, start, wants))
        got = r.step(entries).double().cpu()
        i = 0
        for e in entries:
            if e.want:
                ref = want[e.req_id][[e.start + w for w in e.want]]
                check(got[i:i + len(e.want)], ref, dtype, f"{what} step {n} request {e.req_id}@{e.start}")
            i += len(e.want)
            fed[e.req_id] = e.start + len(e.tokens)
        for rid in (ends or {}).get(n, ()):
            r.finish(rid)
        r.cache.check()


def runner_for(model_dir, dtype, **kw):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    opts = dict(dtype=dtype, max_model_len=512, max_num_seqs=4, max_num_batched_tokens=256, block_size=16,
                num_blocks=64, max_logits_rows=256, decode_exempt_from_budget=False)
    opts.update(kw)
    return ModelRunner.from_dir(model_dir, EngineOptions(**opts))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_layer_sizes_of_the_large_models(big_models, plain_models, name, dtype):
    pm = plain_models(name)
    a, b = tokens(100, 1), tokens(37, 2)
    want = {"a": pm.forward(a), "b": pm.forward(b)}
    r = runner_for(big_models[name], dtype)
    steps = [[("a", a[:90], list(range(90)))]]
    steps += [[("a", [a[90 + i]], [0])] for i in range(4)]
    steps += [[("a", a[94:], list(range(6))), ("b", b[:30], list(range(30)))], [("b", b[30:], list(range(7)))]]
    run_steps(r, steps, want, dtype, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_large_layer_sizes_many_decoding_beside_portions(big_models, plain_models, name, dtype):
    """Eight live requests, five to seven of them decoding while the others bring prompt portions of 2 to 70 tokens:
    the single rows go through split-K attention, the portions through the prompt kernel, the products see 10 to 80 rows."""
    pm = plain_models(name)
    rng = random.Random(7)
    lens = {k: rng.randrange(60, 150) for k in range(11)}
    prompt = {k: rng.randrange(20, n - 25) for k, n in lens.items()}
    seqs = {k: tokens(n, 50 + k) for k, n in lens.items()}
    want = {k: pm.forward(v) for k, v in seqs.items()}
    pool = sum(sorted(-(-n // 16) for n in lens.values())[-8:]) + 2
    r = runner_for(big_models[name], dtype, max_num_seqs=8, num_blocks=pool, max_model_len=160)
    todo, live, fed, steps, ends, busy = list(seqs), [], {}, [], {}, 0
    while todo or live:
        if todo and len(live) < 8 and (len(steps) % 3 == 0 or not live):
            k = todo.pop(0)
            live.append(k)
            fed[k] = 0
        st, singles, portions = [], 0, 0
        for k in list(live):
            n = 1 if fed[k] >= prompt[k] else min(prompt[k] - fed[k], rng.choice([2, 5, 16, 33, 70]))
            singles += n == 1
            portions += n > 1
            st.append((k, seqs[k][fed[k]:fed[k] + n], list(range(n))))
            fed[k] += n
            if fed[k] == lens[k]:
                live.remove(k)
                ends.setdefault(len(steps), []).append(k)
        busy += singles >= 4 and portions >= 1
        steps.append(st)
    assert busy >= 10, "the schedule must hold steps with four or more single rows beside a portion"
    run_steps(r, steps, want, dtype, f"{name} many live", ends)
    assert r.cache.num_free(0) == r.num_blocks


MANY = [(40, "bfloat16"), (64, "bfloat16"), (64, "float32")]


@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
@pytest.mark.parametrize("num,dtype", MANY)
@pytest.mark.parametrize("name", list(SHAPES))
def test_large_layer_sizes_many_requests_decoding(big_models, plain_models, name, num, dtype, graph):
    """40 and 64 requests decode for 12 steps from prompts of unequal length: beyond 32 rows the products of a step run
    in the vendor library and in the kernel that keeps the activations in LDS, the split-K attention reads its keys
    past the caches and, at 64 requests of 8 kv heads, merges its parts inside a workgroup; with graphs the steps are
    replays of the buckets of 40 and 64 rows. Every decoded row against the plain model."""
    pm = plain_models(name)
    steps_n = 12
    rng = random.Random(num)
    plen = {i: rng.randrange(1, 70) for i in range(num)}
    seqs = {i: tokens(plen[i] + steps_n, 300 + i) for i in range(num)}
    want = {i: pm.forward(v) for i, v in seqs.items()}
    r = runner_for(big_models[name], dtype, max_num_seqs=num, num_blocks=num * 6 + 2, max_model_len=96,
                   max_num_batched_tokens=1024, max_logits_rows=64, hip_graph=graph)
    steps, group = [], []
    for i in range(num):
        group.append((i, seqs[i][:plen[i]], [plen[i] - 1]))
        if len(group) == 16 or i == num - 1:
            steps.append(group)
            group = []
    for s in range(steps_n):
        steps.append([(i, [seqs[i][plen[i] + s]], [0]) for i in range(num)])
    run_steps(r, steps, want, dtype, f"{name} {num} decoding")
    assert bool(r._graphs) == graph


def test_decode_graph_with_library_products_replays_equal_eager(big_models):
    """40 requests decoding: more rows than the weight-streaming kernel takes, so the vendor library's products
    (with the algorithm measured per shape) are inside the captured graph. Every replay is checked against the
    same step run eagerly, with eager steps (another request's prompt portions) between the replays."""
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    rng = random.Random(4)
    B = 40
    prompts = [[rng.randrange(2048) for _ in range(12 + i % 5)] for i in range(B)]
    tail = [[rng.randrange(2048) for _ in range(6)] for _ in range(B)]
    extra = [rng.randrange(2048) for _ in range(90)]
    outs = {}
    for graph in (False, True):
        opt = EngineOptions(dtype="bfloat16", max_model_len=512, max_num_seqs=48, max_num_batched_tokens=1024,
                            block_size=16, num_blocks=256, max_logits_rows=64, decode_exempt_from_budget=False,
                            hip_graph=graph)
        r = ModelRunner.from_dir(big_models["8B"], opt)
        got = []
        entries = []
        for i, p in enumerate(prompts):
            assert r.reserve(i, 0, len(p))
            entries.append(Entry(i, p, 0, [len(p) - 1]))
        got.append(r.step(entries).float().cpu())
        fed_extra = 0
        for s in range(6):
            entries = []
            for i, p in enumerate(prompts):
                assert r.reserve(i, len(p) + s, 1)
                entries.append(Entry(i, [tail[i][s]], len(p) + s, [0]))
            got.append(r.step(entries).float().cpu())                        # the graph's bucket of 48 rows
            assert r.reserve("x", fed_extra, 15)
            got.append(r.step([Entry("x", extra[fed_extra:fed_extra + 15], fed_extra, [14])]).float().cpu())  # eager
            fed_extra += 15
        assert bool(r._graphs) == graph
        outs[graph] = got
    for step, (a, b) in enumerate(zip(outs[False], outs[True])):
        torch.testing.assert_close(b, a, rtol=2e-2, atol=2e-2, msg=lambda m: f"step {step}: {m}")


def test_bfloat16_against_the_32bit_path_at_the_8b_layer_sizes(tmp_path):
    """Four layers of the 8B sizes with a 32k vocabulary: the bfloat16 path (MFMA attention, weight-streaming and
    library products) against the true 32-bit path of the same engine on the same weights. Rows whose best two
    logits lie apart in 32-bit must keep their winner (the reference's rule, models/qwen3/tests/real_parity.rs:58-62,
    129-145), prompt positions and decoded ones alike, and no logit strays by more than a fraction of its row's spread."""
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=32768, head_dim=128, num_hidden_layers=4, rms_norm_eps=1e-6,
               rope_theta=1e6, max_position_embeddings=1024, tie_word_embeddings=False, **SHAPES["8B"])
    write_random_model(Qwen3Config.from_dict(cfg), tmp_path, seed=9)
    rng = random.Random(2)
    toks = [rng.randrange(32768) for _ in range(330)]
    got = {}
    for dtype in ("float32", "bfloat16"):
        opt = EngineOptions(dtype=dtype, max_model_len=1024, max_num_seqs=2, max_num_batched_tokens=512, block_size=16,
                            num_blocks=64, max_logits_rows=512)
        r = ModelRunner.from_dir(tmp_path, opt)
        assert r.reserve("a", 0, 300)
        rows = [r.step([Entry("a", toks[:300], 0, list(range(300)))]).float().cpu()]
        for i in range(300, 330):
            assert r.reserve("a", i, 1)
            rows.append(r.step([Entry("a", [toks[i]], i, [0])]).float().cpu())
        got[dtype] = torch.cat(rows)
        del r
        torch.cuda.empty_cache()
    ref, low = got["float32"], got["bfloat16"]
    spread = ref.std(-1, keepdim=True)
    assert float(((low - ref).abs() / spread).max()) < 0.1
    top2 = ref.topk(2, -1).values
    clear = (top2[:, 0] - top2[:, 1]) > 0.15 * spread[:, 0]
    assert int(clear.sum()) > 100
    assert bool((low.argmax(-1)[clear] == ref.argmax(-1)[clear]).all())


_ONE_STEP = """
import sys, random
import torch
from dinfer_amd.config import EngineOptions
from dinfer_amd.engine.batch import Entry
from dinfer_amd.engine.runner import ModelRunner
model, tuning, plans, out = sys.argv[1:5]
opt = EngineOptions(dtype="bfloat16", max_model_len=512, max_num_seqs=4, max_num_batched_tokens=640, block_size=16,
                    num_blocks=48, max_logits_rows=64, gemm_tuning=tuning, gemm_plan_file=plans)
r = ModelRunner.from_dir(model, opt)
rng = random.Random(11)
ids = [rng.randrange(2048) for _ in range(520)]
assert r.reserve("a", 0, 400) and r.reserve("b", 0, 120)
logits = r.step([Entry("a", ids[:400], 0, list(range(0, 400, 9))), Entry("b", ids[400:], 0, list(range(0, 120, 9)))])
torch.save(logits.cpu(), out)
from dinfer_amd.kernels import blaslt
print("measured" if any(p and p.times for p in blaslt._plans.values()) else "not measured")
"""


@pytest.mark.parametrize("tuning", ["heuristic", "measured"])
def test_two_fresh_processes_compute_the_same_bits(big_models, tmp_path, tuning):
    """A step of 520 rows (a prompt portion beside decoding requests: the products run in the vendor library) in two
    processes started one after the other: the bfloat16 logits are equal bit for bit. With the library's first
    suggestion nothing is measured at all; with measured algorithms the first process measures during its warm-up
    and keeps its choices in the plan file, the second reads them there and measures nothing."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    outs, said = [], []
    for i in range(2):
        out = tmp_path / f"logits{i}.pt"
        p = subprocess.run([sys.executable, "-c", _ONE_STEP, str(big_models["8B"]), tuning, str(tmp_path / "plans.json"),
                            str(out)], capture_output=True, text=True, timeout=600, cwd=str(root))
        assert p.returncode == 0, p.stderr[-2000:]
        outs.append(torch.load(out, weights_only=True))
        said.append(p.stdout.strip().splitlines()[-1])
    assert said == (["not measured", "not measured"] if tuning == "heuristic" else ["measured", "not measured"])
    assert torch.equal(outs[0], outs[1])
    assert outs[0].shape == (45 + 14, VOCAB) and bool(outs[0].isfinite().all())
