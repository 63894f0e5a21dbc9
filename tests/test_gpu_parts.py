"""Each part alone against the plain functions, built from parameters only (no model around it);
and a toy mixer with state of its own, defined here, registered, built and stepped through the
engine without a change to the framework's files."""
import random
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as plain
from dinfer_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def context(dtype=torch.float32, page=8, max_tokens=64):
    from dinfer_amd.parts import BuildContext
    return BuildContext(DEV, dtype, max_tokens, max_tokens, page, max_reqs=4)


def whole_batch(n_tokens_per_req, page=8, groups=1):
    """A batch of whole prompts starting at position 0, with pages from a real cache manager."""
    from dinfer_amd.cache import CacheManager, GroupSpec
    from dinfer_amd.engine.batch import Entry, StepBatch
    cache = CacheManager([GroupSpec(page, 64)] * groups, 4)
    entries = []
    for i, n in enumerate(n_tokens_per_req):
        cache.admit(i)
        cache.allocate(i, 0, n)
        entries.append(Entry(i, [0] * n, 0, []))
    b = StepBatch(DEV, 64, 4, 64, [16] * groups)
    b.fill(entries, cache)
    b.upload()
    return b


def loader(tensors, dtype):
    return lambda name, compute=False: tensors[name].to(DEV).to(dtype)


def tol(dtype):
    return dict(rtol=3e-2, atol=3e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from dinfer_amd.parts import NORMS
    n = NORMS.get("rmsnorm")(width=80, eps=3e-6)
    assert n.tensors()["weight"].shape == (80,)
    w = torch.rand(80) + 0.5
    n.load(loader({"weight": w}, dtype))
    x = torch.randn(7, 80, device=DEV).to(dtype)
    out = torch.empty_like(x)
    n.forward(x, out, 7)
    torch.testing.assert_close(out.double().cpu(), plain.rms_norm(x.double().cpu(), w.to(dtype).double(), 3e-6), **tol(dtype))


def test_position_part_builds_the_table_from_its_parameters():
    from dinfer_amd.parts import POSITION_ENCODINGS
    pe = POSITION_ENCODINGS.get("rotary")(head_dim=48, theta=5e4, max_positions=100, rotary_dim=32)
    pe.bind(context())
    t = pe.table().cpu().double()
    assert t.shape == (100, 32) and pe.rotary_dim == 32 and pe.style == 0
    ang = plain.rope_angles(list(range(100)), 32, 5e4)
    torch.testing.assert_close(t, torch.cat([ang.cos(), ang.sin()], 1), rtol=0, atol=1e-6)
    assert POSITION_ENCODINGS.get("none")(head_dim=48).table() is None
    with pytest.raises(ValueError):
        POSITION_ENCODINGS.get("rotary")(head_dim=48, theta=1e4, max_positions=10, rotary_dim=50)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from dinfer_amd.parts import FEED_FORWARDS
    ff = FEED_FORWARDS.get("gated_mlp")(hidden=80, intermediate=136)
    w = {"gate_proj.weight": torch.randn(136, 80) * 0.1, "up_proj.weight": torch.randn(136, 80) * 0.1,
         "down_proj.weight": torch.randn(80, 136) * 0.1}
    assert {k: v.shape for k, v in ff.tensors().items()} == {k: tuple(v.shape) for k, v in w.items()}
    ff.load(loader(w, dtype))
    ff.bind(context(dtype))
    b = whole_batch([11])
    x = torch.randn(64, 80, device=DEV).to(dtype)
    out = ff.forward(x, b)[:11]
    wd = {k: v.to(dtype).double() for k, v in w.items()}
    want = plain.swiglu_mlp(x[:11].double().cpu(), wd["gate_proj.weight"], wd["up_proj.weight"], wd["down_proj.weight"])
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 5])
def test_attention_part(dtype, window):
    """The mixer alone: projections, per-head norm, rotation, cache write, attention, output projection;
    two requests in one batch; sizes and constants only from its parameters."""
    from dinfer_amd.parts import MIXERS, CacheView, part
    H, Hkv, D, Hd, page, theta, eps = 6, 2, 32, 40, 8, 3e4, 2e-5
    mx = MIXERS.get("attention")(hidden=Hd, heads=H, kv_heads=Hkv, head_dim=D, window=window,
                                 position=part("rotary", theta=theta, max_positions=64),
                                 qk_norm=part("rmsnorm", eps=eps))
    spec = mx.cache_spec()
    assert (spec.kv_heads, spec.head_dim, spec.window) == (Hkv, D, window)
    w = {"q_proj.weight": torch.randn(H * D, Hd) * 0.2, "k_proj.weight": torch.randn(Hkv * D, Hd) * 0.2,
         "v_proj.weight": torch.randn(Hkv * D, Hd) * 0.2, "o_proj.weight": torch.randn(Hd, H * D) * 0.2,
         "q_norm.weight": torch.rand(D) + 0.5, "k_norm.weight": torch.rand(D) + 0.5}
    assert {k: v.shape for k, v in mx.tensors().items()} == {k: tuple(v.shape) for k, v in w.items()}
    mx.load(loader(w, dtype))
    mx.bind(context(dtype, page=page))
    lens = [13, 9]
    b = whole_batch(lens, page=page)
    kc = torch.zeros(ops.k_cache_shape(64, Hkv, page, D), device=DEV, dtype=dtype)
    vc = torch.zeros(64, Hkv, D, page, device=DEV, dtype=dtype)
    x = torch.randn(64, Hd, device=DEV).to(dtype)
    out = mx.forward(x, b, CacheView(0, kc, vc, owner=True))[:sum(lens)].double().cpu()
    cfg = dict(num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=eps, rope_theta=theta)
    wd = {"p." + k: v.to(dtype).double() for k, v in w.items()}
    t0 = 0
    for n in lens:
        want = plain.attention_block(x[t0:t0 + n].double().cpu(), list(range(n)), wd, "p.", cfg, window)
        torch.testing.assert_close(out[t0:t0 + n], want, **tol(dtype))
        t0 += n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_part(dtype):
    """The pre-norm arrangement with the deferred residual adds equals the plain layer."""
    from dinfer_amd.parts import BLOCKS, CacheView, LayerSpec, part
    Hd, H, Hkv, D, I, page = 48, 3, 1, 16, 56, 8
    cfg = dict(num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-5, rope_theta=1e4,
               use_sliding_window=False)
    layer = LayerSpec(block=part("prenorm"), norm=part("rmsnorm", eps=1e-5), prefix="model.layers.0.",
                      mixer=part("attention", heads=H, kv_heads=Hkv, head_dim=D, qk_norm=part("rmsnorm", eps=1e-5),
                                 position=part("rotary", theta=1e4, max_positions=64)),
                      feed_forward=part("gated_mlp", intermediate=I))
    blk = BLOCKS.get("prenorm")(hidden=Hd, layer=layer)
    g = torch.Generator().manual_seed(1)
    w = {n: (torch.rand(s.shape, generator=g) + 0.5) if s.init == "gain" else torch.randn(s.shape, generator=g) * 0.2
         for n, s in blk.tensors().items()}
    blk.load(loader(w, dtype))
    blk.bind(context(dtype, page=page))
    wd = {"model.layers.0." + k: v.to(dtype).double() for k, v in w.items()}
    # 10 tokens: the second norm is carried by the products around it; 40: it is a kernel of its own
    for n in (10, 40):
        b = whole_batch([n], page=page)
        kc = torch.zeros(ops.k_cache_shape(64, Hkv, page, D), device=DEV, dtype=dtype)
        vc = torch.zeros(64, Hkv, D, page, device=DEV, dtype=dtype)
        h0 = torch.randn(64, Hd, generator=g).to(DEV).to(dtype)
        prev = torch.randn(64, Hd, generator=g).to(DEV).to(dtype)       # the previous layer's branch, not yet added
        hidden = h0.clone()
        pending = blk.forward(hidden, prev, b, CacheView(0, kc, vc, owner=True))
        got = (hidden[:n].double() + pending[:n].double()).cpu()
        want = plain.decoder_layer((h0[:n].double() + prev[:n].double()).cpu(), list(range(n)), wd, 0, cfg)
        if dtype == torch.float32:
            torch.testing.assert_close(got, want, **tol(dtype))
        else:
            # a whole layer chains a dozen bf16 roundings: judge the error against the spread of the output. Over two
            # dozen seeds both forms give 0.005 to 0.0063 for the root mean square and 0.02 to 0.035 for the largest.
            err = (got - want).abs()
            assert float(err.pow(2).mean().sqrt() / want.std()) < 0.008, n
            assert float(err.max() / want.std()) < 0.045, n


def test_block_carries_its_norms_into_the_next_block():
    """Two blocks in a row at a few tokens: the first returns a Carried for the second's input norm (no norm kernel
    runs between them), and the stream and the second block's branch equal two plain layers."""
    from dinfer_amd.parts import BLOCKS, CacheView, Carried, LayerSpec, part
    dtype = torch.bfloat16
    Hd, H, Hkv, D, I, page = 80, 5, 1, 16, 104, 8
    cfg = dict(num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-5, rope_theta=1e4,
               use_sliding_window=False)
    g = torch.Generator().manual_seed(5)
    blocks, wd = [], {}
    for i in range(2):
        layer = LayerSpec(block=part("prenorm"), norm=part("rmsnorm", eps=1e-5), prefix=f"model.layers.{i}.",
                          mixer=part("attention", heads=H, kv_heads=Hkv, head_dim=D, qk_norm=part("rmsnorm", eps=1e-5),
                                     position=part("rotary", theta=1e4, max_positions=64)),
                          feed_forward=part("gated_mlp", intermediate=I))
        blk = BLOCKS.get("prenorm")(hidden=Hd, layer=layer)
        w = {n: (torch.rand(s.shape, generator=g) + 0.5) if s.init == "gain" else torch.randn(s.shape, generator=g) * 0.2
             for n, s in blk.tensors().items()}
        blk.load(loader(w, dtype))
        blocks.append(blk)
        wd.update({f"model.layers.{i}." + k: v.to(dtype).double() for k, v in w.items()})
    ctx = context(dtype, page=page)
    for blk in blocks:
        blk.bind(ctx)
    n = 7
    b = whole_batch([n], page=page)
    caches = [CacheView(0, torch.zeros(ops.k_cache_shape(64, Hkv, page, D), device=DEV, dtype=dtype),
                        torch.zeros(64, Hkv, D, page, device=DEV, dtype=dtype), owner=True) for _ in blocks]
    h0 = torch.randn(64, Hd, generator=g).to(DEV).to(dtype)
    hidden = h0.clone()
    carried = blocks[0].forward(hidden, None, b, caches[0], next_norm=blocks[1].input_norm())
    assert isinstance(carried, Carried) and carried.norm is blocks[1].norm_in
    want1 = plain.decoder_layer(h0[:n].double().cpu(), list(range(n)), wd, 0, cfg)
    # the stream is complete: nothing is pending. (Root mean square of the error over the output's spread, over 40
    # seeds: 0.006 at the median and 0.009 at worst after one layer, 0.008 and 0.013 after two, with the norms carried
    # and with norm kernels alike; the largest error after two layers 0.03 and 0.07.)
    err = (hidden[:n].double().cpu() - want1).abs()
    assert float(err.pow(2).mean().sqrt() / want1.std()) < 0.011
    pending = blocks[1].forward(hidden, carried, b, caches[1])
    assert isinstance(pending, torch.Tensor)                 # nobody to carry the next norm: the branch comes back
    got = (hidden[:n].double() + pending[:n].double()).cpu()
    want2 = plain.decoder_layer(want1, list(range(n)), wd, 1, cfg)
    err = (got - want2).abs()
    assert float(err.pow(2).mean().sqrt() / want2.std()) < 0.016 and float(err.max() / want2.std()) < 0.08
    # a consumer that cannot take a Carried gets the norm's own kernel on the stream as it stands
    normed = carried.materialise()[:n].double().cpu()
    hs = hidden[:n].double().cpu()
    gain = wd["model.layers.1.input_layernorm.weight"]
    torch.testing.assert_close(normed, plain.rms_norm(hs, gain, 1e-5), rtol=2e-2, atol=2e-2)


# ---- a toy mixer with state of its own ----------------------------------------------------------------
def register_toy():
    from dinfer_amd.config import ModelConfig, key, register_architecture
    from dinfer_amd.parts import MIXERS, LayerSpec, Mixer, ModelSpec, RunEntry, StateSpec, TensorSpec, part

    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + x_t (per request, float32 state in its slot); y_t = s_t W^T."""

        def __init__(self, hidden, decay):
            self.hidden, self.decay = hidden, decay

        def cache_spec(self):
            return StateSpec((self.hidden,), "float32")

        def tensors(self):
            return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

        def load(self, get):
            self.w = get("mix.weight", compute=True)

        def bind(self, ctx):
            self.out = ctx.workspace.buffer("toy_out", self.hidden)

        def forward(self, x, batch, cache):
            slots = batch.state_slots[:batch.num_reqs].tolist()
            t = 0
            for slot, n in zip(slots, batch.q_lens):
                s = cache.state[slot]
                for i in range(n):
                    s.mul_(self.decay).add_(x[t + i].float())
                    self.out[t + i] = (s @ self.w.float().T).to(self.out.dtype)
                t += n
            return self.out

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int = key(int)
        hidden_size: int = key(int)
        decay: float = key(float)
        ARCHITECTURE = "ToyStateLM"

    def build_spec(c):
        norm = part("rmsnorm", eps=1e-6)
        ff = part("gated_mlp", intermediate=2 * c.hidden_size)
        attn = part("attention", heads=2, kv_heads=1, head_dim=16, position=part("rotary", theta=1e4, max_positions=256))
        layers = [LayerSpec(part("prenorm", mixer_prefix="toy."), part("toy_decay", decay=c.decay), ff, norm, "layers.0."),
                  LayerSpec(part("prenorm"), attn, ff, norm, "layers.1.")]
        # the stateful layer runs twice (shared weights, a state of its own each time), around the attention layer
        return ModelSpec("ToyStateLM", c.vocab_size, c.hidden_size, 256, layers, [RunEntry(0), RunEntry(1), RunEntry(0)],
                         norm, "norm.", "embed.weight", "head.weight", tie_embeddings=True)

    if "toy_decay" not in MIXERS:
        MIXERS.register("toy_decay", DecayMixer)
    register_architecture("ToyStateLM", ToyConfig, build_spec)
    return ToyConfig


def toy_plain(w, ids, decay, dtype):
    """The toy model for one whole sequence, straight torch in float64."""
    Hd = w["embed.weight"].shape[1]
    W = {k: v.double() for k, v in w.items()}
    h = W["embed.weight"][ids]

    def ffn(p, x):
        return plain.swiglu_mlp(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])

    def toy_layer(h):
        p = "layers.0."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], 1e-6)
        s, ys = torch.zeros(Hd, dtype=torch.float64), []
        for t in range(len(ids)):
            s = decay * s + x[t]
            ys.append(s @ W[p + "toy.mix.weight"].T)
        h = h + torch.stack(ys)
        return h + ffn(p, plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], 1e-6))

    def attn_layer(h):
        p = "layers.1."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], 1e-6)
        T = len(ids)
        q = (x @ W[p + "self_attn.q_proj.weight"].T).view(T, 2, 16)
        k = (x @ W[p + "self_attn.k_proj.weight"].T).view(T, 1, 16)
        v = (x @ W[p + "self_attn.v_proj.weight"].T).view(T, 1, 16)
        ang = plain.rope_angles(list(range(T)), 16, 1e4)
        o = plain.causal_attention(plain.rope_neox(q, ang), plain.rope_neox(k, ang), v, 16 ** -0.5)
        h = h + o.reshape(T, 32) @ W[p + "self_attn.o_proj.weight"].T
        return h + ffn(p, plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], 1e-6))

    h = toy_layer(attn_layer(toy_layer(h)))
    return plain.rms_norm(h, W["norm.weight"], 1e-6) @ W["embed.weight"].T


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    from safetensors.torch import load_file
    from dinfer_amd.config import EngineOptions, unregister_architecture
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.parts import MIXERS
    from dinfer_amd.weights import write_random_model
    ToyConfig = register_toy()
    try:
        cfg = ToyConfig.from_dict(dict(vocab_size=97, hidden_size=24, decay=0.8, architectures=["ToyStateLM"]))
        write_random_model(cfg, tmp_path, seed=4, dtype="float32")
        w = load_file(str(tmp_path / "model.safetensors"))
        assert "layers.0.toy.mix.weight" in w and "layers.1.self_attn.q_proj.weight" in w
        opt = EngineOptions(dtype="float32", max_model_len=128, max_num_seqs=3, max_num_batched_tokens=64,
                            block_size=8, num_blocks=32, max_logits_rows=64, decode_exempt_from_budget=False)
        r = ModelRunner.from_dir(tmp_path, opt)
        assert len(r.state_tensors) == 2 and len(r.group_specs) == 1      # two state entries, one page group
        rng = random.Random(1)
        seqs = {k: [rng.randrange(97) for _ in range(n)] for k, n in (("a", 21), ("b", 30), ("c", 9), ("d", 14))}
        want = {k: toy_plain(w, v, 0.8, torch.float64) for k, v in seqs.items()}
        # a and b interleaved in portions; c afterwards in a's slot (its state must start from zero); d whole
        plan = [[("a", 5), ("b", 2)], [("b", 11)], [("a", 16), ("b", 1)], [("b", 16), ("c", 9)], [("d", 14)]]
        fed = {k: 0 for k in seqs}
        for st in plan:
            entries = []
            for k, n in st:
                assert r.reserve(k, fed[k], n)
                entries.append(Entry(k, seqs[k][fed[k]:fed[k] + n], fed[k], list(range(n))))
            logits = r.step(entries).double().cpu()
            i = 0
            for e in entries:
                n = len(e.tokens)
                torch.testing.assert_close(logits[i:i + n], want[e.req_id][e.start:e.start + n], rtol=1e-4, atol=1e-5)
                i += n
                fed[e.req_id] += n
                if fed[e.req_id] == len(seqs[e.req_id]):
                    r.finish(e.req_id)
        r.cache.check()
    finally:
        unregister_architecture("ToyStateLM")
        MIXERS.unregister("toy_decay")


# ---- a toy feed-forward with routing, another position encoding, and a layer that reads another's cache ------
def register_routed_toy():
    from dinfer_amd.config import ModelConfig, key, register_architecture
    from dinfer_amd.parts import (FEED_FORWARDS, POSITION_ENCODINGS, FeedForward, LayerSpec, ModelSpec,
                                  PositionEncoding, RunEntry, TensorSpec, part)

    class RoutedFF(FeedForward):
        """Every token goes to its top_k of E small gated experts; router logits and their softmax in float32,
        the chosen weights renormalised to sum 1."""

        def __init__(self, hidden, experts, top_k, intermediate):
            self.hidden, self.E, self.k, self.inter = hidden, experts, top_k, intermediate

        def tensors(self):
            t = {"router.weight": TensorSpec((self.E, self.hidden))}
            for e in range(self.E):
                t[f"experts.{e}.gate.weight"] = TensorSpec((self.inter, self.hidden))
                t[f"experts.{e}.up.weight"] = TensorSpec((self.inter, self.hidden))
                t[f"experts.{e}.down.weight"] = TensorSpec((self.hidden, self.inter))
            return t

        def load(self, get):
            self.router = get("router.weight").float()
            self.w = [tuple(get(f"experts.{e}.{n}.weight", compute=True).float() for n in ("gate", "up", "down"))
                      for e in range(self.E)]

        def bind(self, ctx):
            self.out = ctx.workspace.buffer("routed_out", self.hidden)

        def forward(self, x, batch):
            T = batch.num_tokens
            xf = x[:T].float()
            p = torch.softmax(xf @ self.router.T, dim=-1)
            top, idx = p.topk(self.k, dim=-1)
            top = top / top.sum(dim=-1, keepdim=True)
            y = torch.zeros_like(xf)
            for e, (g, u, d) in enumerate(self.w):
                wgt = (top * (idx == e)).sum(dim=-1, keepdim=True)       # 0 for tokens that did not choose e
                y += wgt * ((torch.nn.functional.silu(xf @ g.T) * (xf @ u.T)) @ d.T)
            self.out[:T] = y.to(self.out.dtype)
            return self.out

    class SlowedRotary(PositionEncoding):
        """Rotation of the first rotary_dim dims in interleaved pairs (2i, 2i + 1) by position / factor."""

        def __init__(self, head_dim, theta, max_positions, rotary_dim, factor):
            self.rotary_dim, self.style = rotary_dim, 1
            self.theta, self.max_positions, self.factor = theta, max_positions, factor

        def bind(self, ctx):
            i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
            ang = (torch.arange(self.max_positions, dtype=torch.float64) / self.factor)[:, None] \
                * (self.theta ** (-2.0 * i / self.rotary_dim))[None, :]
            self._table = torch.cat([ang.cos(), ang.sin()], dim=1).float().to(ctx.device)

        def table(self):
            return self._table

    @dataclass(frozen=True)
    class RoutedConfig(ModelConfig):
        vocab_size: int = key(int)
        hidden_size: int = key(int)
        ARCHITECTURE = "ToyRoutedLM"

    def build_spec(c):
        norm = part("rmsnorm", eps=1e-5)
        slowed = part("toy_slowed_rotary", theta=100.0, max_positions=128, rotary_dim=16, factor=4.0)
        layers = [
            LayerSpec(part("prenorm"), part("attention", heads=3, kv_heads=1, head_dim=32, position=slowed),
                      part("toy_routed", experts=4, top_k=2, intermediate=24), norm, "layers.0."),
            LayerSpec(part("prenorm"), part("attention", heads=2, kv_heads=2, head_dim=16, position=part("none"), window=12),
                      part("gated_mlp", intermediate=40), norm, "layers.1."),
        ]
        # the third entry runs layer 0 again on the keys and values the first entry wrote (it writes none)
        run = [RunEntry(0), RunEntry(1), RunEntry(0, cache=0)]
        return ModelSpec("ToyRoutedLM", c.vocab_size, c.hidden_size, 128, layers, run, norm, "norm.", "embed.weight",
                         "head.weight", tie_embeddings=False)

    FEED_FORWARDS.register("toy_routed", RoutedFF)
    POSITION_ENCODINGS.register("toy_slowed_rotary", SlowedRotary)
    register_architecture("ToyRoutedLM", RoutedConfig, build_spec)
    return RoutedConfig


def routed_toy_plain(w, ids):
    """The routed toy model for one whole sequence, straight torch in float64."""
    W = {k: v.double() for k, v in w.items()}
    T = len(ids)
    h = W["embed.weight"][ids]

    def slowed_rope(x):                      # x [T, heads, 32]: dims 0..15 in pairs (2i, 2i + 1), the rest untouched
        i = torch.arange(8, dtype=torch.float64)
        ang = (torch.arange(T, dtype=torch.float64) / 4.0)[:, None] * (100.0 ** (-2.0 * i / 16))[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = x[..., 0:16:2], x[..., 1:16:2]
        y = x.clone()
        y[..., 0:16:2], y[..., 1:16:2] = a * c - b * s, b * c + a * s
        return y

    def routed(p, x):
        pr = torch.softmax(x @ W[p + "router.weight"].T, dim=-1)
        y = torch.zeros_like(x)
        for t in range(T):
            top = sorted(range(4), key=lambda e: (-float(pr[t, e]), e))[:2]
            tot = sum(pr[t, e] for e in top)
            for e in top:
                q = p + f"experts.{e}."
                y[t] += pr[t, e] / tot * plain.swiglu_mlp(x[t:t + 1], W[q + "gate.weight"], W[q + "up.weight"], W[q + "down.weight"])[0]
        return y

    def layer0(h, kv):
        p = "layers.0."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], 1e-5)
        q = slowed_rope((x @ W[p + "self_attn.q_proj.weight"].T).view(T, 3, 32))
        if kv is None:
            kv = (slowed_rope((x @ W[p + "self_attn.k_proj.weight"].T).view(T, 1, 32)),
                  (x @ W[p + "self_attn.v_proj.weight"].T).view(T, 1, 32))
        o = plain.causal_attention(q, kv[0], kv[1], 32 ** -0.5)
        h = h + o.reshape(T, 96) @ W[p + "self_attn.o_proj.weight"].T
        return h + routed(p + "mlp.", plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], 1e-5)), kv

    def layer1(h):
        p = "layers.1."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], 1e-5)
        q, k, v = ((x @ W[p + f"self_attn.{n}_proj.weight"].T).view(T, 2, 16) for n in "qkv")
        h = h + plain.causal_attention(q, k, v, 16 ** -0.5, window=12).reshape(T, 32) @ W[p + "self_attn.o_proj.weight"].T
        x = plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], 1e-5)
        return h + plain.swiglu_mlp(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])

    h, kv = layer0(h, None)
    h, _ = layer0(layer1(h), kv)
    return plain.rms_norm(h, W["norm.weight"], 1e-5) @ W["head.weight"].T


def test_toy_routing_position_encoding_and_shared_cache(tmp_path):
    """A feed-forward that routes, a position encoding of another kind and a run order in which a layer runs
    twice, the second time on the first time's cache: all defined here, no file of the framework changed.
    Two page groups (every key; a window of 12), replayed whole, in portions and token by token."""
    from safetensors.torch import load_file
    from dinfer_amd.config import EngineOptions, unregister_architecture
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.parts import FEED_FORWARDS, POSITION_ENCODINGS
    from dinfer_amd.weights import write_random_model
    RoutedConfig = register_routed_toy()
    try:
        cfg = RoutedConfig.from_dict(dict(vocab_size=113, hidden_size=40, architectures=["ToyRoutedLM"]))
        write_random_model(cfg, tmp_path, seed=9, dtype="float32")
        w = load_file(str(tmp_path / "model.safetensors"))
        assert "layers.0.mlp.experts.3.down.weight" in w and "layers.0.mlp.router.weight" in w
        # make the router decisive, so that float32 and float64 choose the same experts
        from safetensors.torch import save_file
        w["layers.0.mlp.router.weight"] = w["layers.0.mlp.router.weight"] * 40.0
        save_file(w, str(tmp_path / "model.safetensors"))
        opt = EngineOptions(dtype="float32", max_model_len=128, max_num_seqs=3, max_num_batched_tokens=64,
                            block_size=8, num_blocks=24, max_logits_rows=64)
        r = ModelRunner.from_dir(tmp_path, opt)
        assert len(r.group_specs) == 2 and len(r.cache_views) == 3 and not r.cache_views[2].owner
        assert not r.cache.prefix_caching                      # a window group: pages do not outlive their use
        rng = random.Random(3)
        seqs = {k: [rng.randrange(113) for _ in range(n)] for k, n in (("a", 50), ("b", 37), ("c", 22))}
        want = {k: routed_toy_plain(w, v) for k, v in seqs.items()}
        plan = [[("a", 50)], [("b", 7), ("c", 2)], [("b", 1), ("c", 9)], [("b", 13), ("c", 1)], [("b", 16), ("c", 10)]]
        fed = {k: 0 for k in seqs}

        def run(st):
            entries = []
            for k, n in st:
                assert r.reserve(k, fed[k], n)
                entries.append(Entry(k, seqs[k][fed[k]:fed[k] + n], fed[k], list(range(n))))
            logits = r.step(entries).double().cpu()
            i = 0
            for e in entries:
                n = len(e.tokens)
                torch.testing.assert_close(logits[i:i + n], want[e.req_id][e.start:e.start + n], rtol=2e-4, atol=2e-5)
                i += n
                fed[e.req_id] += n
                r.advance(e.req_id, fed[e.req_id])
                if fed[e.req_id] == len(seqs[e.req_id]):
                    r.finish(e.req_id)

        for st in plan:
            run(st)
        fed["a"] = 0                                          # again, token by token, in pages used before
        for _ in range(len(seqs["a"])):
            run([("a", 1)])
        r.cache.check()
        assert r.cache.num_free(0) == 24 and r.cache.num_free(1) == 24
    finally:
        unregister_architecture("ToyRoutedLM")
        FEED_FORWARDS.unregister("toy_routed")
        POSITION_ENCODINGS.unregister("toy_slowed_rotary")


# ---- a norm of another kind and another arrangement of the block -----------------------------------------------
def register_parallel_toy():
    from dinfer_amd.config import ModelConfig, key, register_architecture
    from dinfer_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, LayerSpec, ModelSpec, Norm, RunEntry,
                                  TensorSpec, part)

    class CenteredNorm(Norm):
        """y = (x - mean) / sqrt(var + eps) * weight + bias (with `residual`: residual += x first, rows gathered by `rows`)."""

        def __init__(self, width, eps):
            self.width, self.eps = width, eps

        def tensors(self):
            return {"weight": TensorSpec((self.width,), init="gain"), "bias": TensorSpec((self.width,))}

        def load(self, get):
            self.weight, self.bias = get("weight").float(), get("bias").float()

        def forward(self, x, out, n_rows, *, residual=None, rows=None):
            idx = rows[:n_rows].long() if rows is not None else torch.arange(n_rows, device=x.device)
            v = x[idx].float()
            if residual is not None:
                v = v + residual[idx].float()
                residual[idx] = v.to(residual.dtype)
            c = v - v.mean(-1, keepdim=True)
            out[:n_rows] = (c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias).to(out.dtype)
            return out

    class ParallelBlock(Block):
        """h += mixer(norm(h)) + ff(norm(h)): one norm, both branches read it."""

        def __init__(self, hidden, layer):
            self.hidden = hidden
            self.mixer = MIXERS.get(layer.mixer.kind)(hidden=hidden, **layer.mixer.params)
            self.ff = FEED_FORWARDS.get(layer.feed_forward.kind)(hidden=hidden, **layer.feed_forward.params)
            self.norm = NORMS.get(layer.norm.kind)(hidden, **layer.norm.params)
            self._parts = (("attn.", self.mixer), ("ff.", self.ff), ("ln.", self.norm))

        def tensors(self):
            return {p + n: s for p, part_ in self._parts for n, s in part_.tensors().items()}

        def load(self, get):
            for p, part_ in self._parts:
                part_.load(lambda name, _p=p, **kw: get(_p + name, **kw))

        def bind(self, ctx):
            for _, part_ in self._parts:
                part_.bind(ctx)
            self.normed = ctx.workspace.buffer("normed", self.hidden)
            self.both = ctx.workspace.buffer("both_branches", self.hidden)

        def forward(self, hidden, pending, batch, cache):
            T = batch.num_tokens
            self.norm.forward(hidden if pending is None else pending, self.normed, T,
                              residual=None if pending is None else hidden)
            a = self.mixer.forward(self.normed, batch, cache)
            f = self.ff.forward(self.normed, batch)
            self.both[:T] = a[:T] + f[:T]
            return self.both

    @dataclass(frozen=True)
    class ParallelConfig(ModelConfig):
        vocab_size: int = key(int)
        hidden_size: int = key(int)
        layers: int = key(int)
        ARCHITECTURE = "ToyParallelLM"

    def build_spec(c):
        norm = part("toy_centered", eps=1e-5)
        attn = part("attention", heads=4, kv_heads=2, head_dim=16, position=part("rotary", theta=1e4, max_positions=128))
        layers = [LayerSpec(part("toy_parallel"), attn, part("gated_mlp", intermediate=56), norm, f"blocks.{i}.")
                  for i in range(c.layers)]
        return ModelSpec("ToyParallelLM", c.vocab_size, c.hidden_size, 128, layers, [RunEntry(i) for i in range(c.layers)],
                         norm, "ln_f.", "wte.weight", "head.weight", tie_embeddings=True)

    NORMS.register("toy_centered", CenteredNorm)
    BLOCKS.register("toy_parallel", ParallelBlock)
    register_architecture("ToyParallelLM", ParallelConfig, build_spec)
    return ParallelConfig


def parallel_toy_plain(w, ids, layers):
    W = {k: v.double() for k, v in w.items()}
    T = len(ids)
    h = W["wte.weight"][ids]

    def ln(x, p):
        c = x - x.mean(-1, keepdim=True)
        return c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + 1e-5) * W[p + "weight"] + W[p + "bias"]

    for i in range(layers):
        p = f"blocks.{i}."
        x = ln(h, p + "ln.")
        q = (x @ W[p + "attn.q_proj.weight"].T).view(T, 4, 16)
        k = (x @ W[p + "attn.k_proj.weight"].T).view(T, 2, 16)
        v = (x @ W[p + "attn.v_proj.weight"].T).view(T, 2, 16)
        ang = plain.rope_angles(list(range(T)), 16, 1e4)
        o = plain.causal_attention(plain.rope_neox(q, ang), plain.rope_neox(k, ang), v, 16 ** -0.5)
        a = o.reshape(T, 64) @ W[p + "attn.o_proj.weight"].T
        f = plain.swiglu_mlp(x, W[p + "ff.gate_proj.weight"], W[p + "ff.up_proj.weight"], W[p + "ff.down_proj.weight"])
        h = h + a + f
    return ln(h, "ln_f.") @ W["wte.weight"].T


def test_toy_norm_and_block_arrangement(tmp_path):
    """A norm that centres and has a bias, and a block whose two branches read one norm and are added together:
    both defined here, registered, built from a configuration and stepped (whole, in portions, token by token,
    the last step asking for the logits of a few rows only, which the final norm then gathers)."""
    from safetensors.torch import load_file
    from dinfer_amd.config import EngineOptions, unregister_architecture
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.parts import BLOCKS, NORMS
    from dinfer_amd.weights import write_random_model
    Config = register_parallel_toy()
    try:
        cfg = Config.from_dict(dict(vocab_size=89, hidden_size=48, layers=3, architectures=["ToyParallelLM"]))
        write_random_model(cfg, tmp_path, seed=2, dtype="float32")
        w = load_file(str(tmp_path / "model.safetensors"))
        assert "blocks.2.ln.bias" in w and "ln_f.bias" in w and "head.weight" not in w
        opt = EngineOptions(dtype="float32", max_model_len=128, max_num_seqs=2, max_num_batched_tokens=64, block_size=8,
                            num_blocks=16, max_logits_rows=64)
        r = ModelRunner.from_dir(tmp_path, opt)
        rng = random.Random(6)
        a = [rng.randrange(89) for _ in range(41)]
        b = [rng.randrange(89) for _ in range(23)]
        want = {"a": parallel_toy_plain(w, a, 3), "b": parallel_toy_plain(w, b, 3)}
        seqs = {"a": a, "b": b}
        fed = {"a": 0, "b": 0}
        plan = [[("a", 30, None)], [("a", 1, None), ("b", 9, None)], [("a", 1, None), ("b", 1, None)],
                [("a", 9, [0, 8]), ("b", 13, [12])]]
        for st in plan:
            entries = []
            for k, n, wants in st:
                assert r.reserve(k, fed[k], n)
                entries.append(Entry(k, seqs[k][fed[k]:fed[k] + n], fed[k], list(range(n)) if wants is None else wants))
            logits = r.step(entries).double().cpu()
            i = 0
            for e in entries:
                for j in e.want:
                    torch.testing.assert_close(logits[i], want[e.req_id][e.start + j], rtol=2e-4, atol=2e-5)
                    i += 1
                fed[e.req_id] += len(e.tokens)
        assert fed == {"a": 41, "b": 23}
    finally:
        unregister_architecture("ToyParallelLM")
        NORMS.unregister("toy_centered")
        BLOCKS.unregister("toy_parallel")


# ---- what a model does to its embeddings and to its logits is a matter of its spec -------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_operations_on_the_embeddings_and_the_logits(tmp_path, dtype):
    """An architecture whose embeddings are multiplied by the root of the width and by a learned vector (a stream
    operation defined here, with a tensor of its own in the weight file) and whose logits are softly capped (the
    built-in one): both are named in its spec; DecoderModel is not touched. Whole, in portions, decoding from graphs."""
    from dataclasses import dataclass as dc
    from safetensors.torch import load_file
    from dinfer_amd.config import EngineOptions, ModelConfig, key, register_architecture, unregister_architecture
    from dinfer_amd.engine.batch import Entry
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.parts import STREAM_OPS, LayerSpec, ModelSpec, Part, RunEntry, TensorSpec, part
    from dinfer_amd.weights import write_random_model

    class LearnedScale(Part):
        """x = x * scale * gain, gain a vector of the file."""

        def __init__(self, width, scale):
            self.width, self.scale = width, scale

        def tensors(self):
            return {"gain": TensorSpec((self.width,), init="gain")}

        def load(self, get):
            self.gain = get("gain")

        def forward(self, x, rows):
            x[:rows] = (x[:rows].float() * self.scale * self.gain.float()).to(x.dtype)

    @dc(frozen=True)
    class CappedConfig(ModelConfig):
        vocab_size: int = key(int)
        hidden_size: int = key(int)
        layers: int = key(int)
        cap: float = key(float)
        ARCHITECTURE = "ToyCappedLM"

    def build_spec(c):
        norm = part("rmsnorm", eps=1e-6)
        attn = part("attention", heads=4, kv_heads=2, head_dim=16, position=part("rotary", theta=1e4, max_positions=128),
                    qk_norm=norm)
        layers = [LayerSpec(part("prenorm"), attn, part("gated_mlp", intermediate=72), norm, f"model.layers.{i}.")
                  for i in range(c.layers)]
        return ModelSpec("ToyCappedLM", c.vocab_size, c.hidden_size, 128, layers, [RunEntry(i) for i in range(c.layers)],
                         norm, "model.norm.", "model.embed_tokens.weight", "lm_head.weight", tie_embeddings=False,
                         embed_post=part("toy_learned_scale", scale=c.hidden_size ** 0.5),
                         logits_post=part("scale_softcap", scale=20.0, softcap=c.cap))

    STREAM_OPS.register("toy_learned_scale", LearnedScale)
    register_architecture("ToyCappedLM", CappedConfig, build_spec)
    try:
        cfg = CappedConfig.from_dict(dict(vocab_size=211, hidden_size=40, layers=2, cap=3.0, architectures=["ToyCappedLM"]))
        write_random_model(cfg, tmp_path, seed=8, dtype="float32")
        w = {k: v.double() for k, v in load_file(str(tmp_path / "model.safetensors")).items()}
        assert "model.embed_tokens.weight.post.gain" in w
        pcfg = dict(num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-6, rope_theta=1e4,
                    num_hidden_layers=2)

        def want(ids):
            h = plain.embedding(ids, w["model.embed_tokens.weight"]) * 40 ** 0.5 * w["model.embed_tokens.weight.post.gain"]
            for l in range(2):
                h = plain.decoder_layer(h, list(range(len(ids))), w, l, pcfg)
            z = plain.rms_norm(h, w["model.norm.weight"], 1e-6) @ w["lm_head.weight"].T
            return 3.0 * torch.tanh(20.0 * z / 3.0)

        opt = EngineOptions(dtype=dtype, max_model_len=128, max_num_seqs=2, max_num_batched_tokens=64, block_size=8,
                            num_blocks=32, max_logits_rows=64, hip_graph=True)
        r = ModelRunner.from_dir(tmp_path, opt)
        rng = random.Random(3)
        ids = [rng.randrange(211) for _ in range(50)]
        ref = want(ids)
        assert float(ref.abs().max()) > 2.0 and float(ref.abs().max()) < 3.0, "the cap is felt"
        got, fed = [], 0
        for n in (30, 7, 1, 1, 1, 1, 1, 8):
            assert r.reserve("a", fed, n)
            rows = list(range(n)) if n > 1 else [0]
            got.append(r.step([Entry("a", ids[fed:fed + n], fed, rows)]).double().cpu())
            fed += n
        got = torch.cat(got)
        assert r._graphs, "the single rows were replayed from a graph, the operations inside it"
        if dtype == "float32":
            torch.testing.assert_close(got, ref, rtol=2e-4, atol=2e-5)
        else:
            assert float(((got - ref).abs() / ref.std(-1, keepdim=True)).max()) < 0.08
    finally:
        unregister_architecture("ToyCappedLM")
        STREAM_OPS.unregister("toy_learned_scale")
