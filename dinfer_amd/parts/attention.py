"""Grouped-query attention over the paged cache, with optional per-head q/k
norm, a position encoding and an optional sliding window.

Order of operations (models/qwen3/src/model.rs:199-315): fused q|k|v projection ->
per-head norm of q and k -> rotation -> k, v into the cache pages -> causal
attention over the pages (scale given, default head_dim^-0.5) -> output projection.
"""
from __future__ import annotations

import torch

from ..kernels import attention as attn_kernels
from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS, NORMS, POSITION_ENCODINGS
from .spec import KVSpec, PartSpec, TensorSpec


@MIXERS.register("attention")
class Attention(Mixer):
    carries_norms = True   # the q/k/v product takes a Carried, the output product an Into

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, position: PartSpec,
                 qk_norm: PartSpec | None = None, window: int | None = None, scale: float | None = None):
        if heads % kv_heads:
            raise ValueError(f"heads {heads} not divisible by kv_heads {kv_heads}")
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.window = window
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.q_size, self.kv_size = heads * head_dim, kv_heads * head_dim
        self.qkv = Linear(hidden, self.q_size + 2 * self.kv_size)
        self.o = Linear(self.q_size, hidden)
        self.position = POSITION_ENCODINGS.get(position.kind)(head_dim=head_dim, **position.params)
        self.q_norm = self.k_norm = None
        if qk_norm is not None:
            cls = NORMS.get(qk_norm.kind)
            self.q_norm, self.k_norm = cls(head_dim, **qk_norm.params), cls(head_dim, **qk_norm.params)

    def cache_spec(self):
        return KVSpec(self.kv_heads, self.head_dim, self.window)

    def tensors(self):
        H, D, Hd = self.hidden, self.head_dim, self.hidden
        t = {
            "q_proj.weight": TensorSpec((self.q_size, Hd)),
            "k_proj.weight": TensorSpec((self.kv_size, Hd)),
            "v_proj.weight": TensorSpec((self.kv_size, Hd)),
            "o_proj.weight": TensorSpec((Hd, self.q_size)),
        }
        if self.q_norm is not None:
            t["q_norm.weight"] = TensorSpec((D,), init="gain")
            t["k_norm.weight"] = TensorSpec((D,), init="gain")
        return t

    def load(self, get):
        # q, k, v rows concatenated into one [(H + 2 Hkv) D, hidden] operand (model.rs:141-165)
        self.qkv.set_weight(torch.cat([get("q_proj.weight", compute=True), get("k_proj.weight", compute=True),
                                       get("v_proj.weight", compute=True)], dim=0))
        self.o.set_weight(get("o_proj.weight", compute=True))
        if self.q_norm is not None:
            self.q_norm.load(lambda n, **kw: get("q_norm." + n, **kw))
            self.k_norm.load(lambda n, **kw: get("k_norm." + n, **kw))

    def bind(self, ctx):
        ws = ctx.workspace
        self.page_size = ctx.page_size
        self.position.bind(ctx)
        self.qkv_buf = ws.buffer("qkv", self.q_size + 2 * self.kv_size)
        self.attn_buf = ws.buffer("attn", self.q_size)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.attn_ws = attn_kernels.Workspace(ctx, self.heads, self.kv_heads, self.head_dim)

    def forward(self, x, batch, cache: CacheView, into=None):
        T = batch.num_tokens
        g = cache.group
        self.qkv.forward(x, self.qkv_buf, T, scratch=True)
        qn = self.q_norm
        ops.qkv_post(
            self.qkv_buf, T, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim,
            q_off=0, k_off=self.q_size, v_off=self.q_size + self.kv_size,
            q_gain=qn.weight if qn else None, k_gain=self.k_norm.weight if qn else None,
            eps=qn.eps if qn else 0.0, gain_offset=qn.weight_offset if qn else 0.0,
            positions=batch.positions, cos_sin=self.position.table(), rotary_dim=self.position.rotary_dim,
            rope_style=self.position.style, k_cache=cache.k, v_cache=cache.v,
            slot_mapping=batch.slot_mapping[g] if cache.owner else None, page_size=self.page_size,
            token_runs=batch.max_q_len >= 8)
        attn_kernels.paged_attention(
            self.qkv_buf, self.attn_buf, cache.k, cache.v, batch, g, self.attn_ws, scale=self.scale,
            window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim,
            page_size=self.page_size)
        if into is not None:
            done = self.o.forward_into(self.attn_buf, into, T)
            if done is not None:
                return done
        return self.o.forward(self.attn_buf, self.out_buf, T, scratch=True)
