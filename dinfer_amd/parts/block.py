"""Block arrangements.

"prenorm":  h += mixer(norm_in(h));  h += ff(norm_post(h))
(models/qwen3/src/model.rs:708-813). The feed-forward's add is deferred into the
next block's input norm kernel, and the mixer's add into this block's second
norm kernel, so each add costs no pass of its own (model.rs:700-701,722-731,772-781).
"""
from __future__ import annotations

from .base import Block, CacheView
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from .spec import LayerSpec


def _sub(get, prefix):
    return lambda name, **kw: get(prefix + name, **kw)


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """params: mixer_prefix, ff_prefix, norm_in_name, norm_post_name (weight-name pieces)."""

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

    def tensors(self):
        return {p + n: s for p, part in self._parts() for n, s in part.tensors().items()}

    def load(self, get):
        for p, part in self._parts():
            part.load(_sub(get, p))

    def bind(self, ctx):
        for _, part in self._parts():
            part.bind(ctx)
        self.normed = ctx.workspace.buffer("normed", self.hidden)

    def forward(self, hidden, pending, batch, cache: CacheView):
        T = batch.num_tokens
        if pending is None:
            self.norm_in.forward(hidden, self.normed, T)
        else:
            self.norm_in.forward(pending, self.normed, T, residual=hidden)
        a = self.mixer.forward(self.normed, batch, cache)
        self.norm_post.forward(a, self.normed, T, residual=hidden)
        return self.ff.forward(self.normed, batch)
