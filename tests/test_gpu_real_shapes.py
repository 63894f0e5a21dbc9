"""Four layers of the Qwen3-8B, 14B and 32B sizes (the 8B with its whole vocabulary of 151,936) replayed through
bin/trace_run in the four ways a trace can be cut, in true 32-bit and in bfloat16, against the plain model.

One trace per (sizes, dtype) holds all four ways one after the other, so the model is loaded once a dtype:
  w      a request whole: one step, logits everywhere
  t      most of a request in one step, its last 32 tokens one by one
  p      portions of changing size, down to two tokens and one
  a..g   mixed: up to four live, portions of some beside single tokens of others
The pool (--max-tokens 320: twenty pages) is smaller than what the trace feeds in total, so every way after the
first runs on pages that earlier requests have used.

The plain model runs in float64 with torch's own operations on the GPU. 32-bit bound: the engine sums every product
in float in a fixed order, so a logit carries the rounding of sums of up to K terms (K up to 25,600) through four
layers and the head; measured 2 to 4 e-5 of a row's spread, the bound is `8 eps sqrt(K) (layers + 1)` with
eps = 2^-24, which is 3.8e-4 at the 32B sizes. bfloat16 by the reference's rule (models/qwen3/tests/real_parity.rs:
58-62,129-145): rows whose best two logits lie clearly apart keep their winner; and the error of a row stays a small
fraction of its spread: root mean square below `0.0125 sqrt(layers)` (roundings to 8 bits add up like a random walk
over the layers: measured 0.009 sqrt(layers) at these sizes with two and with four layers), no single logit further
off than 7 times its row's root mean square error (a row of 151,936 logits has entries at 5 of them by chance; a
product tile gone wrong stands out by far more)."""
import json
import math
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
LAYERS = 4

# name -> (sizes, vocabulary)
SHAPES = {
    "8B-4layers-vocab151936": (dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                                    intermediate_size=12288), 151936),
    "14B-4layers-vocab3001": (dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                                   intermediate_size=17408), 3001),
    "32B-4layers-vocab3001": (dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                                   intermediate_size=25600), 3001),
}


def build_trace(vocab, every):
    """(steps, places, sequences): places[step] lists the (request, position) of each wanted row.
    every: of the rows of long portions only every `every`-th is wanted (a row of the whole vocabulary is 0.6 MB)."""
    rng = random.Random(vocab)
    seq = lambda n: [rng.randrange(vocab) for _ in range(n)]
    seqs = {"w": seq(150), "t": seq(150), "p": seq(150)}
    seqs.update({k: seq(n) for k, n in (("a", 70), ("b", 41), ("c", 9), ("d", 55), ("e", 64), ("f", 1), ("g", 37))})
    steps, places = [], {}

    def add(entries, ends):
        i = len(steps)
        out = []
        for rid, start, toks, want in entries:
            out.append({"id": rid, "tokens": toks, "want": want})
            places.setdefault(i, []).extend((rid, start + w) for w in want)
        if not places.get(i):
            places.pop(i, None)
        steps.append({"step": i, "entries": out, "end": ends})

    thin = lambda n: [j for j in range(n) if j % every == 0 or j == n - 1]
    add([("w", 0, seqs["w"], thin(150))], ["w"])
    add([("t", 0, seqs["t"][:118], [117])], [])
    for pos in range(118, 150):
        add([("t", pos, [seqs["t"][pos]], [0])], ["t"] if pos == 149 else [])
    pos, sizes, k = 0, [7, 16, 2, 5, 3, 33, 2, 8, 1], 0
    while pos < 150:
        n = min(sizes[k % len(sizes)], 150 - pos)
        add([("p", pos, seqs["p"][pos:pos + n], thin(n))], ["p"] if pos + n == 150 else [])
        pos, k = pos + n, k + 1
    todo, live, fed = list("abcdefg"), [], {}
    while todo or live:
        while todo and len(live) < 4:
            live.append(todo.pop(0))
            fed[live[-1]] = 0
        entries, ends = [], []
        for r in list(live):
            left = len(seqs[r]) - fed[r]
            if fed[r] > 0 and left <= 12:
                n = 1
            elif rng.random() < 0.2 and fed[r] > 0:
                continue                                         # left out of this step, goes on later
            else:
                n = min(left, rng.choice([2, 3, 5, 8, 13, 16, 21]))
            entries.append((r, fed[r], seqs[r][fed[r]:fed[r] + n], thin(n)))
            fed[r] += n
            if fed[r] == len(seqs[r]):
                ends.append(r)
                live.remove(r)
        add(entries, ends)
    return steps, places, seqs


@pytest.fixture(scope="module", params=list(SHAPES))
def real_model(request, tmp_path_factory):
    """(name, folder, {request: plain logits float64 on the CPU at the wanted positions}, trace)."""
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.weights import write_random_model
    name = request.param
    sizes, vocab = SHAPES[name]
    cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=vocab, head_dim=128, num_hidden_layers=LAYERS,
               rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=40960, tie_word_embeddings=False, **sizes)
    d = tmp_path_factory.mktemp("real_" + name.split("-")[0])
    write_random_model(Qwen3Config.from_dict(cfg), d, seed=len(name))
    steps, places, seqs = build_trace(vocab, every=6 if vocab > 100000 else 1)
    wanted = {}
    for ps in places.values():
        for rid, pos in ps:
            wanted.setdefault(rid, []).append(pos)
    pcfg, w = plain.load(d, dtype=torch.float32)
    w = {k: v.cuda().double() for k, v in w.items()}
    ref = {}
    with torch.device("cuda"):
        for rid, ids in seqs.items():
            ref[rid] = dict(zip(wanted[rid], plain.forward(pcfg, w, ids)[wanted[rid]].cpu()))
    del w
    torch.cuda.empty_cache()
    yield name, d, ref, (steps, places), sizes, vocab


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_ways_of_cutting_at_real_layer_sizes(real_model, tmp_path, dtype):
    name, model_dir, ref, (steps, places), sizes, vocab = real_model
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(tmp_path), "--max-tokens", "320"], input=text, capture_output=True, text=True,
                       timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    bound32 = 8 * 2.0 ** -24 * math.sqrt(sizes["intermediate_size"]) * (LAYERS + 1)
    worst, worst_rms, clear_rows = 0.0, 0.0, 0
    for i, ps in places.items():
        got = torch.from_numpy(np.fromfile(tmp_path / f"{i}.f32", dtype="<f4").reshape(len(ps), vocab)).double()
        want = torch.stack([ref[rid][pos] for rid, pos in ps])
        spread = want.std(-1, keepdim=True)
        err = ((got - want).abs() / spread).max(-1).values
        worst = max(worst, float(err.max()))
        where = f"{name} {dtype} step {i} {ps[int(err.argmax())]}"
        if dtype == "float32":
            assert float(err.max()) < bound32, f"{where}: off by {float(err.max()):.2e} of the row's spread (bound {bound32:.2e})"
        else:
            row_rms = (got - want).pow(2).mean(-1).sqrt() / spread[:, 0]
            rms = float(row_rms.max())
            worst_rms = max(worst_rms, rms)
            assert rms < 0.0125 * math.sqrt(LAYERS), f"{where}: a row is off by {rms:.4f} row-sigmas (root mean square)"
            assert bool((err < 7 * row_rms).all()), f"{where}: one logit is off by {float(err.max()):.3f} row-sigmas"
            top2 = want.topk(2, -1).values
            clear = (top2[:, 0] - top2[:, 1]) > 0.25 * spread[:, 0]
            clear_rows += int(clear.sum())
            assert bool((got.argmax(-1)[clear] == want.argmax(-1)[clear]).all()), f"{where}: argmax differs on a clear row"
    print(f"[real shapes] {name} {dtype}: worst {worst:.2e} (rms {worst_rms:.2e}) of a row's spread over "
          f"{sum(len(v) for v in places.values())} rows, {clear_rows} clear rows", flush=True)
    if dtype == "bfloat16":
        assert clear_rows >= 20
