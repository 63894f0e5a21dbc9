"""The engine against the plain implementation: whole prompts, decoding after a prompt,
portions of changing size, mixed batches with reused pages; 32-bit and bfloat16."""
import random

import pytest
import torch

import plain_qwen3 as plain
from tiny_configs import CONFIGS, PAGE

pytestmark = pytest.mark.gpu

# 32-bit path against the float64 plain model: rounding only.
F32_TOL = dict(rtol=2e-4, atol=2e-5)


def make_runner(model_dir, name, dtype, max_tokens=2048, num_blocks=None, max_seqs=4, max_len=None):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    cfg = CONFIGS[name][0]
    opt = EngineOptions(dtype=dtype, max_model_len=max_len or cfg["max_position_embeddings"], max_num_seqs=max_seqs,
                        max_num_batched_tokens=max_tokens, block_size=PAGE[name], num_blocks=num_blocks or 256,
                        max_logits_rows=max_tokens, decode_exempt_from_budget=False, hip_graph=False)
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
        assert err < 0.08, f"{what}: bf16 logits off by {err:.3f} row-sigmas"
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
