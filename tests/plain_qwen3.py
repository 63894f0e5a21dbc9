"""A plain, slow implementation of Qwen3 dense for whole sequences: no cache, no
paging, no batching, one function per part, written from the reference's
formulas (each function cites where the reference computes the same thing).
It shares no code with ``dinfer_amd``: it reads config.json with ``json`` and the
weights with the ``safetensors`` package.

Everything is computed in the dtype given (float64 by default), so that it can
judge the engine's 32-bit path; it does not imitate bfloat16 roundings.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch


# ---- parts ---------------------------------------------------------------------------------------
def embedding(ids, table):
    """h[t] = E[id_t]  (crates/kernels/cuda/activation.cu:121-129, models/qwen3/src/model.rs:699)."""
    return table[torch.as_tensor(ids, dtype=torch.long)]


def rms_norm(x, w, eps):
    """y = x / sqrt(mean(x^2) + eps) * w; the weight multiplies directly, no 1 + w
    (crates/kernels/cuda/rmsnorm_core.cuh:63-81, norm.cu:99-113)."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x / torch.sqrt(ms + eps) * w


def rope_angles(positions, head_dim, theta, dtype=torch.float64):
    """angle[p, i] = p * theta^(-2i / D), i < D/2  (crates/layers/src/nn.rs:152-185)."""
    i = torch.arange(head_dim // 2, dtype=torch.float64)
    freq = torch.tensor(float(theta), dtype=torch.float64) ** (-2.0 * i / head_dim)
    return (torch.as_tensor(positions, dtype=torch.float64)[:, None] * freq[None, :]).to(dtype)


def rope_neox(x, angles):
    """x [T, heads, D]; pairs (i, i + D/2): a' = a cos - b sin, b' = b cos + a sin
    (crates/kernels/cuda/qkv_post.cu:65-76)."""
    half = x.shape[-1] // 2
    a, b = x[..., :half], x[..., half:]
    c, s = angles.cos()[:, None, :], angles.sin()[:, None, :]
    return torch.cat([a * c - b * s, b * c + a * s], dim=-1)


def causal_attention(q, k, v, scale, window=None):
    """q [T, H, D], k and v [T, Hkv, D] of one whole sequence. Query head h reads kv head
    h // (H / Hkv); row i sees keys j <= i (and j > i - window with a window); softmax over
    scale * q.k; output [T, H, D]
    (crates/kernels/cuda/gqa.cu:1044-1048,1064-1117; models/qwen3/src/model.rs:232)."""
    T, H, D = q.shape
    G = H // k.shape[1]
    out = torch.zeros_like(q)
    for h in range(H):
        kh, vh = k[:, h // G], v[:, h // G]
        s = (q[:, h] @ kh.T) * scale
        i = torch.arange(T)[:, None]
        j = torch.arange(T)[None, :]
        hidden = j > i
        if window is not None:
            hidden = hidden | (j <= i - window)
        s = s.masked_fill(hidden, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ vh
    return out


def silu(x):
    """x / (1 + exp(-x))  (crates/kernels/cuda/common.cuh:55)."""
    return x / (1.0 + torch.exp(-x))


def swiglu_mlp(x, w_gate, w_up, w_down):
    """down( silu(x Wg^T) * (x Wu^T) )  (crates/layers/src/nn.rs:288-311,373-381,
    crates/kernels/cuda/activation.cu:8-16)."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def attention_block(x, positions, w, prefix, cfg, window):
    """q/k/v projections, per-head RMSNorm of q and k (not v) with one gain vector for all
    heads, rotation, attention, output projection (models/qwen3/src/model.rs:141-172,211-313;
    crates/kernels/cuda/qkv_post.cu:48-64)."""
    T = x.shape[0]
    H, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (x @ w[prefix + "q_proj.weight"].T).view(T, H, D)
    k = (x @ w[prefix + "k_proj.weight"].T).view(T, Hkv, D)
    v = (x @ w[prefix + "v_proj.weight"].T).view(T, Hkv, D)
    q = rms_norm(q, w[prefix + "q_norm.weight"], cfg["rms_norm_eps"])
    k = rms_norm(k, w[prefix + "k_norm.weight"], cfg["rms_norm_eps"])
    ang = rope_angles(positions, D, cfg["rope_theta"], x.dtype)
    q, k = rope_neox(q, ang), rope_neox(k, ang)
    o = causal_attention(q, k, v, D ** -0.5, window)
    return o.reshape(T, H * D) @ w[prefix + "o_proj.weight"].T


def layer_window(cfg, layer):
    """Layers from max_window_layers on use the window when use_sliding_window is set
    (the reference refuses the option, models/qwen3/src/config.rs:48; the meaning is the keys')."""
    if cfg.get("use_sliding_window") and layer >= cfg["max_window_layers"]:
        return cfg["sliding_window"]
    return None


def decoder_layer(h, positions, w, layer, cfg):
    """h += Attn(RMSNorm_in(h)); h += MLP(RMSNorm_post(h))  (models/qwen3/src/model.rs:708-813)."""
    p = f"model.layers.{layer}."
    eps = cfg["rms_norm_eps"]
    h = h + attention_block(rms_norm(h, w[p + "input_layernorm.weight"], eps), positions, w, p + "self_attn.", cfg,
                            layer_window(cfg, layer))
    h = h + swiglu_mlp(rms_norm(h, w[p + "post_attention_layernorm.weight"], eps), w[p + "mlp.gate_proj.weight"],
                       w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return h


def forward(cfg, w, ids, first_position=0):
    """Logits [T, V] at every position of one whole sequence
    (models/qwen3/src/model.rs:684-853: embed, layers, final norm, lm_head; the head is
    lm_head.weight if the file has it, else the embedding table, model.rs:487-496)."""
    h = embedding(ids, w["model.embed_tokens.weight"])
    positions = list(range(first_position, first_position + len(ids)))
    for l in range(cfg["num_hidden_layers"]):
        h = decoder_layer(h, positions, w, l, cfg)
    h = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return h @ head.T


def load(model_dir, dtype=torch.float64):
    """(config dict, {name: tensor in dtype}) of a model folder."""
    from safetensors.torch import load_file
    d = Path(model_dir)
    cfg = json.loads((d / "config.json").read_text())
    w = {}
    for f in sorted(d.glob("*.safetensors")):
        w.update({k: v.to(dtype) for k, v in load_file(str(f)).items()})
    return cfg, w


# ---- sampling ------------------------------------------------------------------------------------
M0, M1, W0, W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
MASK = 0xFFFFFFFF


def philox4x32_10(counter, key):
    """Philox4x32 with 10 rounds by its definition (Salmon et al., "Parallel random numbers:
    as easy as 1, 2, 3"); the reference's copy is crates/kernels/cuda/sampling.cu:137-157."""
    c0, c1, c2, c3 = counter
    k0, k1 = key
    for _ in range(10):
        p0, p1 = M0 * c0, M1 * c2
        hi0, lo0, hi1, lo1 = p0 >> 32, p0 & MASK, p1 >> 32, p1 & MASK
        c0, c1, c2, c3 = (hi1 ^ c1 ^ k0) & MASK, lo1, (hi0 ^ c3 ^ k1) & MASK, lo0
        k0, k1 = (k0 + W0) & MASK, (k1 + W1) & MASK
    return c0, c1, c2, c3


def uniform(seed, offset):
    """u in [0, 1): counter = (offset, 0, 0), key = seed, (c0 >> 8) * 2^-24 (sampling.cu:145-157)."""
    c = philox4x32_10((offset & MASK, (offset >> 32) & MASK, 0, 0), (seed & MASK, (seed >> 32) & MASK))
    return (c[0] >> 8) / 16777216.0


def apply_penalties(logits, prompt, output, repetition=1.0, frequency=0.0, presence=0.0):
    """repetition over prompt and output tokens (divide positive, multiply negative logits),
    frequency * count and presence over output tokens (crates/kernels/cuda/sampling.cu:318-349)."""
    z = logits.clone()
    for t in set(prompt) | set(output):
        v = z[t]
        if repetition != 1.0:
            v = v / repetition if v > 0 else v * repetition
        c = output.count(t)
        if c > 0:
            v = v - (frequency * c + presence)
        z[t] = v
    return z


def apply_logit_bias(logits, bias):
    """bias: {token: value} added to the logits before the penalties (crates/kernels/cuda/sampling.cu:286-305)."""
    z = logits.clone()
    for t, b in bias.items():
        z[t] = z[t] + b
    return z


def token_logprobs(logits, chosen, k):
    """(logprob of chosen, rank, [(token, logprob)] of the k most probable) from the log-softmax of the logits as
    the model gave them; rank counts the tokens with a strictly larger logit; equal values go by lower index
    (crates/kernels/cuda/sampling.cu:380-430, crates/core/src/sampler.rs:156-166)."""
    z = logits.double()
    lp = z - torch.logsumexp(z, -1)
    order = sorted(range(z.numel()), key=lambda i: (-float(z[i]), i))[:k]
    return float(lp[chosen]), int((z > z[chosen]).sum()), [(i, float(lp[i])) for i in order]


def candidate_mask(z, top_k=-1, top_p=1.0, min_p=0.0):
    """Which tokens survive min_p -> top-k -> top-p, on z = logits / temperature
    (crates/kernels/cuda/sampling.cu:83-129,352-364; order :266-283). top-p keeps the most
    probable tokens of what top-k left, up to and including the one that crosses p."""
    z = z.clone().double()
    if min_p > 0:
        p = torch.softmax(z, -1)
        z[p < min_p * p.max()] = float("-inf")
    if 0 < top_k < z.numel():
        kth = torch.topk(z, top_k).values[-1]
        z[z < kth] = float("-inf")
    if 0 < top_p < 1:
        srt, idx = torch.sort(z, descending=True)
        cum = torch.softmax(srt, -1).cumsum(-1)
        drop = (cum - torch.softmax(srt, -1)) >= top_p  # mass before this token already reaches p
        z[idx[drop]] = float("-inf")
    return torch.isfinite(z)


def sample_row(logits, temperature, seed, offset, top_k=-1, top_p=1.0, min_p=0.0):
    """One token from one row of logits (crates/kernels/cuda/sampling.cu:159-263):
    temperature <= 1e-5 is argmax with ties to the lowest index; otherwise
    p_i = exp(z_i - max z) over the surviving tokens, target = u * sum p, and the first index in
    vocabulary order whose running sum reaches target. Returns (token, slack) where slack is the
    distance of target from the nearest boundary of the chosen token's interval, relative to the sum."""
    logits = logits.double()
    if temperature <= 1e-5:
        m = logits.max()
        return int((logits == m).nonzero()[0]), 1.0
    z = logits / temperature
    keep = candidate_mask(z, top_k, top_p, min_p)
    p = torch.where(keep, torch.exp(z - z[keep].max()), torch.zeros_like(z))
    cum = p.cumsum(-1)
    target = uniform(seed, offset) * float(cum[-1])
    idx = int(torch.searchsorted(cum, torch.tensor(target, dtype=cum.dtype), right=False))
    idx = min(idx, p.numel() - 1)
    while p[idx] == 0 and idx + 1 < p.numel():
        idx += 1
    lo = float(cum[idx] - p[idx])
    slack = min(target - lo, float(cum[idx]) - target) / float(cum[-1])
    return idx, slack
