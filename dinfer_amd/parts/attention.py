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
    capturable = True      # every kernel reads tokens, positions, slots, tables and lengths from the batch's device buffers
    capturable_portions = True   # the choice of kernels follows the step's counts alone

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, position: PartSpec,
                 qk_norm: PartSpec | None = None, window: int | None = None, scale: float | None = None):
        if heads % kv_heads:
            raise ValueError(f"heads {heads} not divisible by kv_heads {kv_heads}")
        if head_dim <= 0 or head_dim % 8 or head_dim > ops.MAX_HEAD_DIM:   # said at build, not at the first step
            raise ValueError(f"attention: head_dim {head_dim} has no kernel (multiples of 8 up to {ops.MAX_HEAD_DIM}; "
                             "the cache stores keys in pieces of 8 elements)")
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
        for n, spec in self.position.tensors().items():   # an encoding with parameters of its own (rotations have none)
            t["position." + n] = spec
        return t

    def load(self, get):
        # q, k, v rows concatenated into one [(H + 2 Hkv) D, hidden] operand (model.rs:141-165)
        self.qkv.set_weight(torch.cat([get("q_proj.weight", compute=True), get("k_proj.weight", compute=True),
                                       get("v_proj.weight", compute=True)], dim=0))
        self.o.set_weight(get("o_proj.weight", compute=True))
        if self.q_norm is not None:
            self.q_norm.load(lambda n, **kw: get("q_norm." + n, **kw))
            self.k_norm.load(lambda n, **kw: get("k_norm." + n, **kw))
        self.position.load(lambda n, **kw: get("position." + n, **kw))

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
        qn, pos = self.q_norm, self.position
        geometry = dict(heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim, q_off=0, k_off=self.q_size,
                        v_off=self.q_size + self.kv_size, positions=batch.positions, page_size=self.page_size)
        norm = dict(q_gain=qn.weight if qn else None, k_gain=self.k_norm.weight if qn else None,
                    eps=qn.eps if qn else 0.0, gain_offset=qn.weight_offset if qn else 0.0)
        no_norm = dict(q_gain=None, k_gain=None, eps=0.0, gain_offset=0.0)
        write = dict(k_cache=cache.k, v_cache=cache.v, slot_mapping=batch.slot_mapping[g] if cache.owner else None,
                     token_runs=batch.max_q_len >= 8)
        if (pos.fused and batch.all_decode and self.attn_ws.decode_takes_post and pos.style == 0
                and pos.rotary_dim == self.head_dim and (qn is None or qn.weight.dtype == torch.bfloat16)):
            # only single rows: norm, rotation and cache write ride in the attention kernel, one launch fewer a layer
            attn_kernels.decode_with_post(
                self.qkv_buf, self.attn_buf, cache.k, cache.v, batch, g, self.attn_ws, write=cache.owner,
                scale=self.scale, window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads,
                head_dim=self.head_dim, page_size=self.page_size, q_off=0, k_off=self.q_size,
                v_off=self.q_size + self.kv_size, positions=batch.positions, cos_sin=pos.table(), **norm)
            return self._project_out(T, into)
        if pos.fused:
            # per-head norm, rotation by the encoding's table and the cache write in one kernel
            ops.qkv_post(self.qkv_buf, T, **geometry, **norm, cos_sin=pos.table(), rotary_dim=pos.rotary_dim,
                         rope_style=pos.style, **write)
        else:
            # an encoding that is no rotation by a table works on q and k itself, between the norm and the cache write
            if qn:
                ops.qkv_post(self.qkv_buf, T, **geometry, **norm, cos_sin=None, rotary_dim=0, rope_style=0, k_cache=None,
                             v_cache=None, slot_mapping=None, token_runs=False)
            q = self.qkv_buf[:T, :self.q_size].view(T, self.heads, self.head_dim)
            k = self.qkv_buf[:T, self.q_size:self.q_size + self.kv_size].view(T, self.kv_heads, self.head_dim)
            pos.transform(q, k, batch.positions[:T])
            if cache.owner:
                ops.qkv_post(self.qkv_buf, T, **geometry, **no_norm, cos_sin=None, rotary_dim=0, rope_style=0, **write)
        attn_kernels.paged_attention(
            self.qkv_buf, self.attn_buf, cache.k, cache.v, batch, g, self.attn_ws, scale=self.scale,
            window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim,
            page_size=self.page_size)
        return self._project_out(T, into)

    def _project_out(self, T, into):
        if into is not None:
            done = self.o.forward_into(self.attn_buf, into, T)
            if done is not None:
                return done
        return self.o.forward(self.attn_buf, self.out_buf, T, scratch=True)
