"""Contexts of thousands of tokens through the whole model, at the lengths the measurements run at: two layers of the
Qwen3-8B sizes against the plain model in float64 (torch's own operations, on the GPU).

  * one prompt of 4,500 tokens whole and then 32 tokens one by one, through bin/trace_run, in true 32-bit and in
    bfloat16: the prompt kernel's waves walk more than 64 pages each, the rotation table is read up to row 4,531,
    the split-K decode kernel cuts 4,500 keys into dozens of parts that a kernel of its own merges;
  * 64 requests brought to 2,048..2,100 tokens in portions of 512 (four requests' portions a step), then decoding
    eight tokens each together, eagerly and from a captured graph: two parts a request of more than 64 pages each,
    joined inside a workgroup, keys read past the caches (what a decode step of 64 requests of a serving load runs).

With random weights a row's attention over thousands of keys is nearly their mean, and a key that is skipped or read
from a wrong page moves a logit by less than any bound. So the gains of the per-head q norm are made four times
larger in the model folder: scores spread four times wider and a few keys, anywhere in the context, carry each row
(one key read wrongly then changes the row by a large fraction of its size).

Bounds as in test_gpu_real_shapes.py: 32-bit `8 eps sqrt(K) (layers + 1)` of a row's spread; bfloat16 by the
reference's rule (models/qwen3/tests/real_parity.rs:58-62,129-145: rows whose best two logits lie clearly apart keep
their winner), no logit further off than 7 times its row's root-mean-square error, and that error below
`0.0125 sqrt(layers)` of the row's spread times the factor by which the gains were enlarged: a relative error e of
a layer's input (the roundings of the layers before it) moves that layer's scores by e times the size of q, so what
the roundings of bfloat16 make of a row grows with that factor in any implementation (the row at position 0, whose
attention is its own value whatever the scores, stays at the figure of the other files). A key read from a wrong
page moves a row by about its whole spread.
"""
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
LAYERS, VOCAB = 2, 3001
SIZES = dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, intermediate_size=12288)
SHARP = 4.0


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """(folder, plain config, float64 weights on the GPU)."""
    from safetensors.torch import load_file, save_file
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=VOCAB, head_dim=128, num_hidden_layers=LAYERS,
               rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=8192, tie_word_embeddings=False, **SIZES)
    d = tmp_path_factory.mktemp("long_8B")
    write_random_model(Qwen3Config.from_dict(cfg), d, seed=41)
    tensors = load_file(str(d / "model.safetensors"))
    for name in tensors:
        if name.endswith("self_attn.q_norm.weight"):
            tensors[name] = (tensors[name].float() * SHARP).to(tensors[name].dtype)
    save_file(tensors, str(d / "model.safetensors"))
    pcfg, w = plain.load(d, dtype=torch.float32)
    w = {k: v.cuda().double() for k, v in w.items()}
    yield d, pcfg, w
    del w
    torch.cuda.empty_cache()


def plain_rows(pcfg, w, ids, rows):
    with torch.device("cuda"):
        return plain.forward(pcfg, w, ids)[rows].cpu()


def judge(got, want, dtype, what):
    """got, want: [rows, vocab] float64 on the CPU. Returns the number of rows whose winner is clear."""
    spread = want.std(-1, keepdim=True)
    err = ((got - want).abs() / spread).max(-1).values
    if dtype == "float32":
        bound = 8 * 2.0 ** -24 * math.sqrt(SIZES["intermediate_size"]) * (LAYERS + 1)
        assert float(err.max()) < bound, f"{what}: row {int(err.argmax())} off by {float(err.max()):.2e} of its spread (bound {bound:.2e})"
        return 0
    row_rms = (got - want).pow(2).mean(-1).sqrt() / spread[:, 0]
    assert float(row_rms.max()) < 0.0125 * math.sqrt(LAYERS) * SHARP, \
        f"{what}: row {int(row_rms.argmax())} is off by {float(row_rms.max()):.4f} row-sigmas (root mean square)"
    assert bool((err < 7 * row_rms).all()), f"{what}: one logit is off by {float(err.max()):.3f} row-sigmas"
    top2 = want.topk(2, -1).values
    clear = (top2[:, 0] - top2[:, 1]) > 0.25 * spread[:, 0]
    assert bool((got.argmax(-1)[clear] == want.argmax(-1)[clear]).all()), f"{what}: argmax differs on a clear row"
    return int(clear.sum())


def test_sharpened_attention_rests_on_few_keys(long_model):
    """The premise of this file: in the plain model with the enlarged q gains, the largest softmax weight of a late
    row is a sizeable share of the whole, so no row is a mean of thousands of keys."""
    d, pcfg, w = long_model
    rng = random.Random(1)
    ids = [rng.randrange(VOCAB) for _ in range(2100)]
    with torch.device("cuda"):
        h = plain.embedding(ids, w["model.embed_tokens.weight"])
        p = "model.layers.0."
        x = plain.rms_norm(h, w[p + "input_layernorm.weight"], pcfg["rms_norm_eps"])
        H, Hkv, D = 32, 8, 128
        q = plain.rms_norm((x @ w[p + "self_attn.q_proj.weight"].T).view(-1, H, D), w[p + "self_attn.q_norm.weight"], 1e-6)
        k = plain.rms_norm((x @ w[p + "self_attn.k_proj.weight"].T).view(-1, Hkv, D), w[p + "self_attn.k_norm.weight"], 1e-6)
        ang = plain.rope_angles(list(range(len(ids))), D, pcfg["rope_theta"])
        q, k = plain.rope_neox(q, ang), plain.rope_neox(k, ang)
        s = torch.einsum("hd,thd->ht", q[-1], k.repeat_interleave(H // Hkv, 1)) * D ** -0.5
        top = torch.softmax(s, -1).max(-1).values
    assert float(top.median()) > 0.05, f"largest weight among 2,100 keys: median over heads {float(top.median()):.3f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_4500_tokens_then_decoding_through_trace_run(long_model, tmp_path, dtype):
    d, pcfg, w = long_model
    rng = random.Random(5)
    n_prompt, n_decode = 4500, 32
    ids = [rng.randrange(VOCAB) for _ in range(n_prompt + n_decode)]
    wanted = [j for j in range(n_prompt) if j % 64 == 0 or j == n_prompt - 1]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:n_prompt], "want": wanted}], "end": []}]
    for i in range(n_decode):
        steps.append({"step": i + 1, "entries": [{"id": "a", "tokens": [ids[n_prompt + i]], "want": [0]}],
                      "end": ["a"] if i == n_decode - 1 else []})
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", dtype, "--out",
                        str(tmp_path), "--max-tokens", str(n_prompt + n_decode)], input=text, capture_output=True,
                       text=True, timeout=900)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    rows = wanted + list(range(n_prompt, n_prompt + n_decode))
    want = plain_rows(pcfg, w, ids, rows).double()
    read = lambda i, n: torch.from_numpy(np.fromfile(tmp_path / f"{i}.f32", dtype="<f4").reshape(n, VOCAB)).double()
    got = torch.cat([read(0, len(wanted))] + [read(i + 1, 1) for i in range(n_decode)])
    clear = judge(got[:len(wanted)], want[:len(wanted)], dtype, f"{dtype} prompt rows")
    clear += judge(got[len(wanted):], want[len(wanted):], dtype, f"{dtype} decoded rows")
    if dtype == "bfloat16":
        assert clear >= 10


@pytest.mark.parametrize("dtype,graph", [("bfloat16", True), ("bfloat16", False), ("float32", False)],
                         ids=["bfloat16-graph", "bfloat16-eager", "float32-eager"])
def test_64_requests_of_2048_tokens_decoding_together(long_model, dtype, graph):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    d, pcfg, w = long_model
    num, n_decode, portion = 64, 8, 512
    rng = random.Random(64)
    plen = [rng.randrange(2048, 2101) for _ in range(num)]
    seqs = [[rng.randrange(VOCAB) for _ in range(plen[i] + n_decode)] for i in range(num)]
    pages = sum(-(-(n + n_decode) // 16) for n in plen) + 2
    opt = EngineOptions(dtype=dtype, max_model_len=2176, max_num_seqs=num, max_num_batched_tokens=4 * portion,
                        block_size=16, num_blocks=pages, max_logits_rows=num, decode_exempt_from_budget=False,
                        hip_graph=graph)
    r = ModelRunner.from_dir(d, opt)
    got = {i: [] for i in range(num)}
    fed = [0] * num
    # prompts: four requests' portions a step; the row after a prompt's last token is wanted
    for first in range(0, num, 4):
        group = list(range(first, min(first + 4, num)))
        while any(fed[i] < plen[i] for i in group):
            entries = []
            for i in group:
                n = min(portion, plen[i] - fed[i])
                if n <= 0:
                    continue
                assert r.reserve(i, fed[i], n)
                entries.append(Entry(i, seqs[i][fed[i]:fed[i] + n], fed[i], [n - 1] if fed[i] + n == plen[i] else []))
            out = r.step(entries).double().cpu()
            k = 0
            for e in entries:
                fed[e.req_id] = e.start + len(e.tokens)
                r.advance(e.req_id, fed[e.req_id])
                if e.want:
                    got[e.req_id].append(out[k])
                    k += 1
    for s in range(n_decode):
        entries = []
        for i in range(num):
            assert r.reserve(i, plen[i] + s, 1)
            entries.append(Entry(i, [seqs[i][plen[i] + s]], plen[i] + s, [0]))
        out = r.step(entries).double().cpu()
        for i in range(num):
            got[i].append(out[i])
            r.advance(i, plen[i] + s + 1)
    assert bool(r._graphs) == graph
    clear = 0
    for i in range(num):
        rows = list(range(plen[i] - 1, plen[i] + n_decode))
        clear += judge(torch.stack(got[i]), plain_rows(pcfg, w, seqs[i], rows).double(), dtype, f"{dtype} request {i}")
    if dtype == "bfloat16":
        assert clear >= 50
    del r
    torch.cuda.empty_cache()
