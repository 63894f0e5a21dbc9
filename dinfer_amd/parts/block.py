"""Block arrangements.

"prenorm":  h += mixer(norm_in(h));  h += ff(norm_post(h))
(models/qwen3/src/model.rs:708-813). The feed-forward's add is deferred into the
next block's input norm kernel, and the mixer's add into this block's second
norm kernel, so each add costs no pass of its own (model.rs:700-701,722-731,772-781).
In steps of a few tokens the norms have no kernel at all: the product before a norm adds
into the stream and leaves what the norm needs, the product after it applies it (Carried).
In steps of many tokens the product before a norm adds into the stream as well (the library's
beta = 1), and the norm's kernel reads the stream alone.
"""
from __future__ import annotations

import torch

from ..kernels import gemm
from .base import Block, CacheView, Carried, Into
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from .spec import LayerSpec

# A norm is carried by the products around it in steps of up to this many tokens (one token tile of the few-row
# kernel). Measured at the 8B sizes: a step of 1 token 3.82 -> 3.68 ms, of 8 4.07 -> 4.00, of 16 4.65 -> 4.62; at 32
# tokens (two token tiles) the longer ends of four kernels cost more than the two norm kernels did (5.93 -> 6.11 ms);
# carrying only the norm after the mixer there (the down projection has another kernel at those rows) 5.39 -> 5.44 ms,
# and with the kernel for wide weights as the gate/up product that applies it 5.22 -> 5.28 (4.88 -> 4.92 at 24 tokens).
CARRY_ROWS = 16


def _sub(get, prefix):
    return lambda name, **kw: get(prefix + name, **kw)


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """params: mixer_prefix, ff_prefix, norm_in_name, norm_post_name (weight-name pieces)."""
    carries_norms = True

    def __init__(self, hidden: int, layer: LayerSpec, mixer_prefix: str = "self_attn.", ff_prefix: str = "mlp.",
                 norm_in: str = "input_layernorm.", norm_post: str = "post_attention_layernorm."):
        self.hidden = hidden
        self.prefixes = (mixer_prefix, ff_prefix, norm_in, norm_post)
        self.mixer = MIXERS.get(layer.mixer.kind)(hidden=hidden, **layer.mixer.params)
        self.ff = FEED_FORWARDS.get(layer.feed_forward.kind)(hidden=hidden, **layer.feed_forward.params)
        ncls = NORMS.get(layer.norm.kind)
        self.norm_in, self.norm_post = ncls(hidden, **layer.norm.params), ncls(hidden, **layer.norm.params)

    def _parts(self):
        return zip(self.prefixes, (self.mixer, self.ff, self.norm_in, self.norm_post))

    @property
    def capturable(self):
        return all(part.capturable for _, part in self._parts())

    @property
    def capturable_portions(self):
        return all(part.capturable and part.capturable_portions for _, part in self._parts())

    def tensors(self):
        return {p + n: s for p, part in self._parts() for n, s in part.tensors().items()}

    def load(self, get):
        for p, part in self._parts():
            part.load(_sub(get, p))

    def bind(self, ctx):
        for _, part in self._parts():
            part.bind(ctx)
        ws = ctx.workspace
        self.normed = ws.buffer("normed", self.hidden)
        # for norms carried by the products around them (steps of up to CARRY_ROWS tokens)
        self.xg = ws.buffer("carried_xg", self.hidden, rows=CARRY_ROWS)
        self.stats = ws.buffer("carried_stats", -(-self.hidden // gemm.STATS_COLUMNS), dtype=torch.float32,
                               rows=CARRY_ROWS)

    def input_norm(self):
        return self.norm_in if self.mixer.carries_norms else None

    def _into(self, hidden, norm, part, T):
        if norm is None or not part.carries_norms:
            return {}
        return {"into": Into(hidden, norm, self.xg, self.stats, self.normed)}

    def forward(self, hidden, pending, batch, cache: CacheView, next_norm=None):
        T = batch.num_tokens
        if isinstance(pending, Carried):
            x = pending if self.mixer.carries_norms else pending.materialise()
        elif pending is None:
            x = self.norm_in.forward(hidden, self.normed, T)
        else:
            x = self.norm_in.forward(pending, self.normed, T, residual=hidden)
        a = self.mixer.forward(x, batch, cache, **self._into(hidden, self.norm_post, self.mixer, T))
        if isinstance(a, Carried):
            x = a if self.ff.carries_norms else a.materialise()
        else:
            x = self.norm_post.forward(a, self.normed, T, residual=hidden)
        return self.ff.forward(x, batch, **self._into(hidden, next_norm, self.ff, T))
