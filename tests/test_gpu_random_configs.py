"""Random tiny configurations of the architecture (head sizes the MFMA kernels take and do not take, head
counts and groups, widths and vocabularies that are no powers of two, windows, page sizes, tied and untied
heads): whole prompts, a long portion beside a short one, then decoding beside portions, in 32-bit and in
bfloat16, against the plain implementation. Every size either works or is refused when the engine is built."""
import random
import tempfile

import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu


def random_config(rng, seed):
    H = rng.choice([1, 2, 3, 4, 6, 8, 12])
    Hkv = rng.choice([d for d in (1, 2, 3, 4, 6, 8, 12) if H % d == 0])
    D = rng.choice([16, 32, 48, 64, 80, 96, 112, 128]) if seed % 3 else rng.choice([8, 24, 40, 72])
    L = rng.randint(1, 3)
    window = rng.choice([None, None, 5, 17, 40])
    cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=rng.choice([97, 256, 331, 512, 1000]),
               hidden_size=rng.choice([40, 64, 72, 80, 96, 100, 136, 200]),
               intermediate_size=rng.choice([56, 100, 128, 136, 224, 264]), num_hidden_layers=L,
               num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D,
               rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]), rope_theta=rng.choice([1e4, 5e4, 1e6]),
               max_position_embeddings=256, tie_word_embeddings=rng.random() < 0.5)
    if window:
        cfg.update(use_sliding_window=True, sliding_window=window, max_window_layers=rng.randint(0, L))
    return cfg, rng.choice([4, 8, 16, 24, 32, 64])


def check(got, want, dtype, what):
    got = got.double().cpu()
    if dtype == "float32":
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-5, msg=lambda m: f"{what}: {m}")
    else:
        spread = want.std(dim=-1, keepdim=True)
        err = ((got - want).abs() / spread).max().item()
        rms = ((got - want).pow(2).mean(-1, keepdim=True).sqrt() / spread).max().item()
        assert err < 0.08 and rms < 0.02, f"{what}: bf16 logits off by {err:.3f} (rms {rms:.4f}) row-sigmas"


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration(seed):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.weights import write_random_model
    rng = random.Random(1000 + seed)
    cfg, page = random_config(rng, seed)
    what = f"seed {seed}: {cfg} page {page}"
    with tempfile.TemporaryDirectory() as d:
        write_random_model(Qwen3Config.from_dict(cfg), d, seed=seed)
        pc, w = plain.load(d)
        V = cfg["vocab_size"]
        a, b = ([rng.randrange(V) for _ in range(n)] for n in (rng.randint(20, 90), rng.randint(3, 40)))
        want = [plain.forward(pc, w, a), plain.forward(pc, w, b)]
        for dtype in ("float32", "bfloat16"):
            opt = EngineOptions(dtype=dtype, max_model_len=256, max_num_seqs=4, max_num_batched_tokens=256,
                                block_size=page, num_blocks=64, max_logits_rows=256, hip_graph=seed % 2 == 0)
            r = ModelRunner.from_dir(d, opt)
            for i, x in enumerate((a, b)):                       # whole prompts, all positions
                assert r.reserve(i, 0, len(x))
                check(r.step([Entry(i, x, 0, list(range(len(x))))]), want[i], dtype, what)
                r.finish(i)
            na = len(a) - 8                                     # a long portion beside a short one
            assert r.reserve("a", 0, na) and r.reserve("b", 0, 2)
            got = r.step([Entry("a", a[:na], 0, [na - 1]), Entry("b", b[:2], 0, [1])])
            check(got, torch.stack([want[0][na - 1], want[1][1]]), dtype, what)
            pa, pb = na, 2
            while pa < len(a) or pb < len(b):                   # decoding beside portions of changing size
                es, ws = [], []
                if pa < len(a):
                    assert r.reserve("a", pa, 1)
                    es.append(Entry("a", [a[pa]], pa, [0]))
                    ws.append(want[0][pa])
                    pa += 1
                if pb < len(b):
                    n = min(rng.choice([1, 1, 2, 3, 7]), len(b) - pb)
                    assert r.reserve("b", pb, n)
                    es.append(Entry("b", b[pb:pb + n], pb, [n - 1]))
                    ws.append(want[1][pb + n - 1])
                    pb += n
                got = r.step(es)
                for e in es:
                    r.advance(e.req_id, e.start + len(e.tokens))
                check(got, torch.stack(ws), dtype, what)
            r.finish("a")
            r.finish("b")
            r.cache.check()
            assert r.cache.num_free(0) == 64
