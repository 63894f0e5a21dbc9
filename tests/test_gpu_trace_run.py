"""bin/trace_run as a user runs it: a subprocess fed JSON lines, logits read from files."""
import json
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


def run_trace(model_dir, dtype, out_dir, max_tokens, steps):
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", str(max_tokens)], input=text, capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    return p


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_trace_run_mixed(model_dirs, tmp_path, name, dtype):
    cfg, w = plain.load(model_dirs[name])
    V = cfg["vocab_size"]
    rng = random.Random(3)
    seqs = {k: [rng.randrange(V) for _ in range(n)] for k, n in (("a", 50), ("b", 90), ("c", 33), ("d", 64), ("e", 20))}
    want = {k: plain.forward(cfg, w, v) for k, v in seqs.items()}
    # a, b, c live first (64 + 128 + 64 = 256 tokens); d and e reuse the pages of a and c
    steps, fed, expect = [], {k: 0 for k in seqs}, {}
    plan = [
        [("a", 30), ("b", 7)], [("a", 20), ("b", 2), ("c", 33)], [("b", 50)], [("b", 1), ("d", 40)],
        [("b", 1), ("d", 2), ("e", 19)], [("b", 29), ("d", 22), ("e", 1)],
    ]
    for i, st in enumerate(plan):
        entries, ends = [], []
        for k, n in st:
            toks = seqs[k][fed[k]:fed[k] + n]
            wants = sorted(set([0, n - 1]))
            entries.append({"id": k, "tokens": toks, "want": wants})
            for j in wants:
                expect.setdefault(i, []).append((k, fed[k] + j))
            fed[k] += n
            if fed[k] == len(seqs[k]):
                ends.append(k)
        steps.append({"step": i, "entries": entries, "end": ends})
    steps.append({"step": len(plan), "entries": [], "end": []})
    run_trace(model_dirs[name], dtype, tmp_path, 256, steps)
    assert not (tmp_path / f"{len(plan)}.f32").exists()
    for i, places in expect.items():
        got = torch.from_numpy(np.fromfile(tmp_path / f"{i}.f32", dtype="<f4").reshape(len(places), V)).double()
        ref = torch.stack([want[k][p] for k, p in places])
        if dtype == "float32":
            torch.testing.assert_close(got, ref, rtol=2e-4, atol=2e-5)
        else:
            err = ((got - ref).abs() / ref.std(-1, keepdim=True)).max().item()
            assert err < 0.08, f"step {i}: {err}"


def test_trace_run_refuses_what_does_not_fit(model_dirs, tmp_path):
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [1] * 100, "want": []}], "end": []}]
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dirs["A"]), "--dtype",
                        "float32", "--out", str(tmp_path), "--max-tokens", "64"], input=json.dumps(steps[0]) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "64" in p.stderr
