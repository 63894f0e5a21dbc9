"""One layer with the layer sizes of Qwen3-8B, 14B and 32B (group sizes 4, 5 and 8; H * D equal to,
and larger than, the hidden size), random weights, against the plain implementation in 32-bit and
in bfloat16: whole prompt, then decoding, then a second request beside it. The vocabulary is cut to
2048 rows, which is no layer size."""
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


@pytest.fixture(scope="module")
def big_models(tmp_path_factory):
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.weights import write_random_model
    out = {}
    for name, sizes in SHAPES.items():
        cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=2048, head_dim=128, num_hidden_layers=1,
                   rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=512, tie_word_embeddings=False, **sizes)
        d = tmp_path_factory.mktemp(f"big_{name}")
        write_random_model(Qwen3Config.from_dict(cfg), d, seed=len(name))
        out[name] = d
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_layer_sizes_of_the_large_models(big_models, name, dtype):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    cfg, w = plain.load(big_models[name], dtype=torch.float32)
    opt = EngineOptions(dtype=dtype, max_model_len=512, max_num_seqs=4, max_num_batched_tokens=256, block_size=16,
                        num_blocks=64, max_logits_rows=256, decode_exempt_from_budget=False)
    r = ModelRunner.from_dir(big_models[name], opt)
    rng = random.Random(1)
    a = [rng.randrange(2048) for _ in range(100)]
    b = [rng.randrange(2048) for _ in range(37)]
    want = {"a": plain.forward(cfg, w, a).double(), "b": plain.forward(cfg, w, b).double()}
    steps = [[("a", a[:90], list(range(90)))]]
    steps += [[("a", [a[90 + i]], [0])] for i in range(4)]
    steps += [[("a", a[94:], list(range(6))), ("b", b[:30], list(range(30)))], [("b", b[30:], list(range(7)))]]
    fed = {"a": 0, "b": 0}
    for st in steps:
        entries = []
        for rid, toks, wants in st:
            assert r.reserve(rid, fed[rid], len(toks))
            entries.append(Entry(rid, toks, fed[rid], wants))
        got = r.step(entries).double().cpu()
        i = 0
        for e in entries:
            ref = want[e.req_id][e.start:e.start + len(e.tokens)]
            g = got[i:i + len(e.tokens)]
            if dtype == "float32":
                # the plain model runs in float32 here (float64 of these sizes is slow): both sides round
                torch.testing.assert_close(g, ref, rtol=2e-3, atol=2e-4)
            else:
                err = ((g - ref).abs() / ref.std(-1, keepdim=True)).max().item()
                assert err < 0.08, f"{name} {e.req_id}@{e.start}: {err:.3f} row-sigmas"
            i += len(e.tokens)
            fed[e.req_id] += len(e.tokens)


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
