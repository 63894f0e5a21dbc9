"""The plain implementation is the judge of the engine, so it is pinned here by what fixes it
besides the reference's text: special cases that reduce to a library routine, invariants, and
known answers. Each check is chosen so that a plausible mistake fails it (noted per test). No GPU."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from tiny_configs import CONFIGS

torch.manual_seed(0)
D64 = torch.float64


# ---- norm ----------------------------------------------------------------------------------------
def test_rms_norm_invariants():
    x = torch.randn(5, 96, dtype=D64) * 3
    eps = 1e-5
    y = plain.rms_norm(x, torch.ones(96, dtype=D64), eps)
    ms = (x * x).mean(-1, keepdim=True)
    torch.testing.assert_close(y * torch.sqrt(ms + eps), x)                       # undoes itself
    torch.testing.assert_close((y * y).mean(-1, keepdim=True), ms / (ms + eps))   # eps inside the root
    w = torch.randn(96, dtype=D64)
    torch.testing.assert_close(plain.rms_norm(x, w, eps), y * w)                  # weight multiplies, no 1 + w
    torch.testing.assert_close(plain.rms_norm(7 * x, w, 0.0), plain.rms_norm(x, w, 0.0))  # scale-free without eps
    assert not torch.allclose(plain.rms_norm(x, w, eps), (x - x.mean(-1, keepdim=True)) / x.std(-1, keepdim=True) * w)


# ---- rotation ------------------------------------------------------------------------------------
def test_rope_pairs_angles_and_sign():
    D, theta = 16, 1e4
    x = torch.randn(3, 2, D, dtype=D64)
    ang = plain.rope_angles([0, 5, 77], D, theta)
    y = plain.rope_neox(x, ang)
    torch.testing.assert_close(y[0], x[0])                                        # position 0 is the identity
    half = D // 2
    # pairs are (i, i + D/2): each keeps its 2-norm (interleaved pairing (2i, 2i+1) would not)
    torch.testing.assert_close(y[..., :half] ** 2 + y[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2)
    # as complex multiplication by e^{i p f_i}, f_i = theta^(-2i/D): pins the angle, the sign and the frequency order
    z = torch.complex(x[..., :half], x[..., half:])
    f = torch.tensor([theta ** (-2 * i / D) for i in range(half)], dtype=D64)
    for r, p in enumerate([0, 5, 77]):
        zr = z[r] * torch.polar(torch.ones(half, dtype=D64), p * f)
        torch.testing.assert_close(torch.cat([zr.real, zr.imag], -1), y[r])
    assert abs(float(ang[1, 0]) - 5.0) < 1e-12 and abs(float(ang[1, -1]) - 5.0 * theta ** (-(D - 2) / D)) < 1e-12


def test_rope_scores_depend_on_distance_only():
    D = 32
    q, k = torch.randn(1, 1, D, dtype=D64), torch.randn(1, 1, D, dtype=D64)
    def score(pq, pk):
        return float((plain.rope_neox(q, plain.rope_angles([pq], D, 1e6)) * plain.rope_neox(k, plain.rope_angles([pk], D, 1e6))).sum())
    assert abs(score(10, 3) - score(110, 103)) < 1e-9
    assert abs(score(10, 3) - score(3, 10)) > 1e-6                                # direction matters


# ---- attention -----------------------------------------------------------------------------------
def test_attention_reduces_to_library_sdpa():
    T, H, D = 9, 4, 16
    q, k, v = (torch.randn(T, H, D, dtype=D64) for _ in range(3))
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(plain.causal_attention(q, k, v, D ** -0.5), want.transpose(0, 1))


def test_attention_groups_window_and_special_cases():
    T, H, Hkv, D = 12, 6, 2, 8
    q, k, v = torch.randn(T, H, D, dtype=D64), torch.randn(T, Hkv, D, dtype=D64), torch.randn(T, Hkv, D, dtype=D64)
    out = plain.causal_attention(q, k, v, 0.3)
    # GQA = MHA with every kv head repeated G times, consecutive query heads sharing one (not strided)
    rep = plain.causal_attention(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), 0.3)
    torch.testing.assert_close(out, rep)
    torch.testing.assert_close(out[0], v[0].repeat_interleave(3, 0))              # one visible key: output is its value
    zero = plain.causal_attention(torch.zeros_like(q), k, v, 0.3)
    torch.testing.assert_close(zero[4, 0], v[:5, 0].mean(0))                      # q = 0: mean of the visible values
    # causality: changing a later token leaves earlier rows alone
    k2, v2 = k.clone(), v.clone()
    k2[7:], v2[7:] = 9.0, -9.0
    torch.testing.assert_close(plain.causal_attention(q, k2, v2, 0.3)[:7], out[:7])
    # window W: row i sees exactly keys i-W+1 .. i
    w = plain.causal_attention(q, k, v, 0.3, window=4)
    torch.testing.assert_close(w[:4], out[:4])
    torch.testing.assert_close(w[9, 0], plain.causal_attention(q[6:10], k[6:10], v[6:10], 0.3)[3, 0])
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=1), v.repeat_interleave(3, 1))


# ---- feed-forward --------------------------------------------------------------------------------
def test_swiglu_against_library_and_special_cases():
    x = torch.randn(4, 10, dtype=D64)
    wg, wu, wd = torch.randn(14, 10, dtype=D64), torch.randn(14, 10, dtype=D64), torch.randn(10, 14, dtype=D64)
    torch.testing.assert_close(plain.silu(x), F.silu(x))
    torch.testing.assert_close(plain.swiglu_mlp(x, wg, wu, wd), (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T)
    assert not torch.allclose(plain.swiglu_mlp(x, wg, wu, wd), plain.swiglu_mlp(x, wu, wg, wd))   # gate is the activated one
    torch.testing.assert_close(plain.swiglu_mlp(x, torch.zeros_like(wg), wu, wd), torch.zeros(4, 10, dtype=D64))


# ---- the whole model -----------------------------------------------------------------------------
@pytest.fixture(scope="module")
def tiny(model_dirs):
    return {n: plain.load(model_dirs[n]) for n in CONFIGS}


def test_model_is_causal_and_shift_invariant(tiny):
    for name, (cfg, w) in tiny.items():
        ids = [(7 * i + 3) % cfg["vocab_size"] for i in range(40)]
        full = plain.forward(cfg, w, ids)
        assert full.shape == (40, cfg["vocab_size"])
        ids2 = ids[:25] + [(t + 1) % cfg["vocab_size"] for t in ids[25:]]
        torch.testing.assert_close(plain.forward(cfg, w, ids2)[:25], full[:25])
        # only distances between positions count: moving the whole sequence changes nothing
        torch.testing.assert_close(plain.forward(cfg, w, ids, first_position=37), full, rtol=1e-9, atol=1e-9)


def test_model_options_matter(tiny):
    """Each configuration key changes the logits, so an engine that ignored one could not pass."""
    cfg, w = tiny["C"]
    ids = [(5 * i + 1) % cfg["vocab_size"] for i in range(60)]
    base = plain.forward(cfg, w, ids)
    for patch in ({"rope_theta": 1e4}, {"rms_norm_eps": 1e-2}, {"sliding_window": 23}, {"max_window_layers": 3},
                  {"use_sliding_window": False}, {"num_hidden_layers": 4}):
        assert not torch.allclose(plain.forward({**cfg, **patch}, w, ids), base, atol=1e-6), patch
    torch.testing.assert_close(plain.forward({**cfg, "sliding_window": 23}, w, ids)[:23], base[:23])
    cfgB, wB = tiny["B"]                                   # untied: the head is its own matrix
    idsB = ids[:10]
    tied = {k: v for k, v in wB.items() if k != "lm_head.weight"}
    assert not torch.allclose(plain.forward(cfgB, tied, idsB), plain.forward(cfgB, wB, idsB))
    cfgA, wA = tiny["A"]                                   # tied: logits are the final hidden state times E^T
    assert "lm_head.weight" not in wA


def variant_forward(cfg, w, ids, first_position=0, mistake=None):
    """The model put together again from the plain parts, with one mistake of composition at a time (None: none, and
    then it must be plain.forward). Used to show that the pins below tell each mistake from the right composition."""
    T, eps = len(ids), cfg["rms_norm_eps"]
    H, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    norm = (lambda x, g: plain.rms_norm(x, 1 + g, eps)) if mistake == "gain_is_one_plus_w" else (lambda x, g: plain.rms_norm(x, g, eps))
    ang = plain.rope_angles(list(range(first_position, first_position + T)), D, cfg["rope_theta"])
    h = plain.embedding(ids, w["model.embed_tokens.weight"])
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        a = p + "self_attn."
        x = h if mistake == "post_norm" else norm(h, w[p + "input_layernorm.weight"])
        q = (x @ w[a + "q_proj.weight"].T).view(T, H, D)
        k = (x @ w[a + "k_proj.weight"].T).view(T, Hkv, D)
        v = (x @ w[a + "v_proj.weight"].T).view(T, Hkv, D)
        gq, gk = w[a + "q_norm.weight"], w[a + "k_norm.weight"]
        if mistake == "rotation_before_norm":
            q, k = norm(plain.rope_neox(q, ang), gq), norm(plain.rope_neox(k, ang), gk)
        elif mistake == "norm_over_all_heads":
            q = norm(q.reshape(T, 1, H * D), gq.repeat(H)).view(T, H, D)
            k = norm(k.reshape(T, 1, Hkv * D), gk.repeat(Hkv)).view(T, Hkv, D)
            q, k = plain.rope_neox(q, ang), plain.rope_neox(k, ang)
        else:
            q, k = plain.rope_neox(norm(q, gq), ang), plain.rope_neox(norm(k, gk), ang)
        if mistake == "v_normed":
            v = norm(v, gk)
        if mistake == "v_rotated":
            v = plain.rope_neox(v, ang)
        o = plain.causal_attention(q, k, v, D ** -0.5, plain.layer_window(cfg, l)).reshape(T, H * D) @ w[a + "o_proj.weight"].T
        h_mid = norm(h + o, w[p + "input_layernorm.weight"]) if mistake == "post_norm" else h + o
        y = h_mid if mistake == "post_norm" else norm(h if mistake == "mlp_reads_the_layer_input" else h_mid,
                                                      w[p + "post_attention_layernorm.weight"])
        m = plain.swiglu_mlp(y, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        h = norm(h_mid + m, w[p + "post_attention_layernorm.weight"]) if mistake == "post_norm" else h_mid + m
    h = norm(h, w["model.norm.weight"])
    return h @ (w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]).T


def pin_shift(f, cfg, w, ids):
    """Only distances between positions count."""
    return torch.allclose(f(cfg, w, ids, 0), f(cfg, w, ids, 37), rtol=1e-9, atol=1e-9)


def pin_single_token(f, cfg, w, ids):
    """A sequence of one token attends to itself alone: its attention is its value row as the projection left it,
    whatever the q and k norms, the rotation and the position are; library operations only."""
    G = cfg["num_attention_heads"] // cfg["num_key_value_heads"]
    D, eps = cfg["head_dim"], cfg["rms_norm_eps"]
    rms = lambda x, g: x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * g
    h = w["model.embed_tokens.weight"][ids[:1]]
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        v = F.linear(rms(h, w[p + "input_layernorm.weight"]), w[p + "self_attn.v_proj.weight"])
        h = h + F.linear(v.view(-1, D).repeat_interleave(G, 0).reshape(1, -1), w[p + "self_attn.o_proj.weight"])
        y = rms(h, w[p + "post_attention_layernorm.weight"])
        h = h + F.linear(F.silu(F.linear(y, w[p + "mlp.gate_proj.weight"])) * F.linear(y, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    want = F.linear(rms(h, w["model.norm.weight"]), w.get("lm_head.weight", w["model.embed_tokens.weight"]))
    return torch.allclose(f(cfg, w, ids[:1], 5), want, rtol=1e-9, atol=1e-9)


def pin_head_scale(f, cfg, w, ids):
    """The q and k norms are per head: making one head's projection rows larger changes nothing (eps aside)."""
    D = cfg["head_dim"]
    cfg0 = {**cfg, "rms_norm_eps": 1e-30}
    w2 = dict(w)
    for l in range(cfg["num_hidden_layers"]):
        a = f"model.layers.{l}.self_attn."
        w2[a + "q_proj.weight"] = w[a + "q_proj.weight"].clone()
        w2[a + "q_proj.weight"][D:2 * D] *= 7.0
        w2[a + "k_proj.weight"] = w[a + "k_proj.weight"].clone()
        w2[a + "k_proj.weight"][:D] *= 0.3
    return torch.allclose(f(cfg0, w2, ids, 0), f(cfg0, w, ids, 0), rtol=1e-8, atol=1e-8)


def pin_silent_branches(f, cfg, w, ids):
    """With output and down projections of zero both branches add nothing: the logits are the final norm of the
    embeddings times the head (the stream passes every layer untouched, and is normed once, at the end)."""
    w2 = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in w.items()}
    h = w["model.embed_tokens.weight"][ids]
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + cfg["rms_norm_eps"]) * w["model.norm.weight"]
    return torch.allclose(f(cfg, w2, ids, 0), F.linear(h, w.get("lm_head.weight", w["model.embed_tokens.weight"])), rtol=1e-9, atol=1e-9)


def pin_zero_gain_silences(f, cfg, w, ids):
    """The gain multiplies (no 1 + w): layer norms with gains of zero feed zeros to both branches."""
    w2 = {k: (torch.zeros_like(v) if k.endswith(("input_layernorm.weight", "post_attention_layernorm.weight")) else v)
          for k, v in w.items()}
    return pin_silent_branches(lambda c, ww, i, p: f(c, w2, i, p), cfg, w, ids)


def test_each_mistake_of_composition_fails_a_pin(tiny):
    """What fixes the composition of a layer besides the reference's text (models/qwen3/src/model.rs:708-813,
    crates/kernels/cuda/qkv_post.cu:48-76; the same formulas a second time in the reference's own Python,
    scripts/verify/gen_kernel_refs.py:289-322): invariants and special cases that reduce to library routines. The
    right composition keeps all of them; each plausible mistake breaks the one named beside it. Two conventions have
    no anchor but those texts: that a gain multiplies as it is (and not as 1 + w), which the last pin spells out, and
    the order of a block (norm, branch, add; the feed-forward reads the stream after attention), which the one-token
    case spells out in library operations. An installed package's model code is no source here and is not imported."""
    pins = {"rotation_before_norm": pin_shift, "v_rotated": pin_shift, "v_normed": pin_single_token,
            "norm_over_all_heads": pin_head_scale, "post_norm": pin_silent_branches,
            "mlp_reads_the_layer_input": pin_single_token, "gain_is_one_plus_w": pin_zero_gain_silences}
    for name, (cfg, w) in tiny.items():
        ids = [(11 * i + 2) % cfg["vocab_size"] for i in range(30)]
        torch.testing.assert_close(variant_forward(cfg, w, ids), plain.forward(cfg, w, ids), rtol=0, atol=0)
        for pin in set(pins.values()):
            assert pin(plain.forward, cfg, w, ids), f"{name}: the plain model breaks {pin.__name__}"
        for mistake, pin in pins.items():
            wrong = lambda c, ww, i, p=0, m=mistake: variant_forward(c, ww, i, p, m)
            assert not torch.allclose(wrong(cfg, w, ids), plain.forward(cfg, w, ids), atol=1e-6), f"{mistake} changes nothing"
            assert not pin(wrong, cfg, w, ids), f"{name}: {mistake} passes {pin.__name__}"


def test_layer_against_a_hand_rolled_single_head_case():
    """One layer, one head, identity-like weights: every step can be followed by hand."""
    Hd = 8
    cfg = dict(num_attention_heads=1, num_key_value_heads=1, head_dim=8, rms_norm_eps=0.0, rope_theta=1e4)
    eye = torch.eye(Hd, dtype=D64)
    w = {"p.q_proj.weight": eye, "p.k_proj.weight": eye, "p.v_proj.weight": 2 * eye, "p.o_proj.weight": eye,
         "p.q_norm.weight": torch.ones(Hd, dtype=D64), "p.k_norm.weight": torch.ones(Hd, dtype=D64)}
    x = torch.randn(1, Hd, dtype=D64)
    out = plain.attention_block(x, [3], w, "p.", cfg, None)
    torch.testing.assert_close(out, 2 * x)                # a single token attends to itself: o = v = 2x


# ---- sampling ------------------------------------------------------------------------------------
def test_philox_known_answers():
    """Philox4x32-10 test vectors of the Random123 distribution (kat_vectors)."""
    assert plain.philox4x32_10((0, 0, 0, 0), (0, 0)) == (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)
    assert plain.philox4x32_10((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2) == (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)
    assert plain.philox4x32_10((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0)) == \
        (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)
    u = [plain.uniform(9, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in u) and abs(sum(u) / 2000 - 0.5) < 0.03
    assert plain.uniform(9, 5) != plain.uniform(10, 5) and plain.uniform(9, 5) == plain.uniform(9, 5)


def test_inverse_cdf_rule_by_hand():
    logits = torch.log(torch.tensor([0.1, 0.2, 0.3, 0.4]))
    # intervals of the running sum: [0, .1] (.1, .3] (.3, .6] (.6, 1]
    seen = set()
    for off in range(200):
        u = plain.uniform(1, off)
        tok, _ = plain.sample_row(logits, 1.0, 1, off)
        assert tok == (0 if u <= 0.1 else 1 if u <= 0.3 else 2 if u <= 0.6 else 3)
        seen.add(tok)
    assert seen == {0, 1, 2, 3}
    assert plain.sample_row(torch.tensor([1.0, 5.0, 5.0, 0.0]), 0.0, 1, 0)[0] == 1   # greedy ties: lowest index
    assert plain.sample_row(logits, 1e-6, 1, 0)[0] == 3


def test_candidate_masks():
    z = torch.log(torch.tensor([0.5, 0.25, 0.15, 0.07, 0.03]))
    assert plain.candidate_mask(z, top_k=2).tolist() == [True, True, False, False, False]
    assert plain.candidate_mask(z, top_p=0.7).tolist() == [True, True, False, False, False]   # .5 + .25 crosses .7
    assert plain.candidate_mask(z, top_p=0.76).tolist() == [True, True, True, False, False]
    assert plain.candidate_mask(z, min_p=0.2).tolist() == [True, True, True, False, False]    # p >= .2 * .5
    # top-p is applied to what top-k left: of {.5, .25} renormalised, .5 / .75 = .667 crosses .6 alone
    assert plain.candidate_mask(z, top_k=2, top_p=0.6).tolist() == [True, False, False, False, False]


def test_penalties_by_hand():
    z = torch.tensor([2.0, -2.0, 1.0, 1.0, 3.0])
    out = plain.apply_penalties(z, prompt=[0, 1], output=[1, 2, 2], repetition=2.0, frequency=0.5, presence=0.1)
    torch.testing.assert_close(out, torch.tensor([1.0, -4.0 - 0.6, 0.5 - 1.1, 1.0, 3.0]))


def test_logit_bias_and_logprobs_by_hand():
    p = torch.tensor([0.5, 0.25, 0.125, 0.125])
    z = torch.log(p) + 3.0                                  # any shift of the logits leaves the probabilities
    lp, rank, top = plain.token_logprobs(z, 2, 3)
    assert abs(lp - math.log(0.125)) < 1e-6 and rank == 2   # two tokens are more probable; its twin is not
    assert [t for t, _ in top] == [0, 1, 2]                 # of the equal pair the lower index comes first
    torch.testing.assert_close(torch.tensor([v for _, v in top], dtype=torch.float64), torch.log(p[:3]).double(), rtol=1e-6, atol=1e-6)
    assert plain.token_logprobs(z, 0, 0) == (pytest.approx(math.log(0.5), abs=1e-6), 0, [])
    # against the library's routine
    g = torch.randn(300, generator=torch.Generator().manual_seed(4)) * 4
    lp, rank, top = plain.token_logprobs(g, 17, 5)
    ref = torch.log_softmax(g.double(), -1)
    assert abs(lp - float(ref[17])) < 1e-12 and [t for t, _ in top] == torch.topk(g, 5).indices.tolist()
    assert rank == int((ref > ref[17]).sum())
    b = plain.apply_logit_bias(torch.tensor([1.0, 2.0, 3.0]), {0: 5.0, 2: -100.0})
    assert b.tolist() == [6.0, 2.0, -97.0]
