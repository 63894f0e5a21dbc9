"""A decoder model assembled from a ModelSpec: embedding (-> an operation on it, if the spec names one) -> run list
of blocks -> final norm on the wanted rows -> LM head (-> an operation on the logits, if the spec names one).
Knows no architecture by name.
"""
from __future__ import annotations

import torch

from ..kernels import gemm, ops
from .base import BuildContext, Carried
from .linear import Linear
from .registry import BLOCKS, NORMS, STREAM_OPS
from .spec import ModelSpec, RunEntry, TensorSpec


def _build_blocks(spec: ModelSpec):
    return [BLOCKS.get(l.block.kind)(hidden=spec.hidden_size, layer=l, **l.block.params) for l in spec.layers]


def _stream_ops(spec: ModelSpec) -> list:
    """[(weight-name prefix, part)] of the operations on the embeddings and on the logits, None where there is none."""
    made = []
    for part, width, prefix in ((spec.embed_post, spec.hidden_size, spec.embed_name), (spec.logits_post, spec.vocab_size, spec.head_name)):
        made.append(None if part is None else (prefix + ".post.", STREAM_OPS.get(part.kind)(width, **part.params)))
    return made


def expected_tensors(spec: ModelSpec, blocks=None) -> tuple[dict[str, TensorSpec], set[str]]:
    """(name -> TensorSpec for every tensor the model reads, names that may be present or absent)."""
    blocks = blocks or _build_blocks(spec)
    exp = {spec.embed_name: TensorSpec((spec.vocab_size, spec.hidden_size))}
    for l, b in zip(spec.layers, blocks):
        for n, s in b.tensors().items():
            exp[l.prefix + n] = s
    fn = NORMS.get(spec.final_norm.kind)(spec.hidden_size, **spec.final_norm.params)
    for n, s in fn.tensors().items():
        exp[spec.final_norm_name + n] = s
    for op in _stream_ops(spec):
        if op is not None:
            for n, ts in op[1].tensors().items():
                exp[op[0] + n] = ts
    optional = set()
    if spec.tie_embeddings:
        # A tied checkpoint may still ship the head; it is used when present (model.rs:487-496).
        optional.add(spec.head_name)
    else:
        exp[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden_size))
    return exp, optional


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.blocks = _build_blocks(spec)
        self.final_norm = NORMS.get(spec.final_norm.kind)(spec.hidden_size, **spec.final_norm.params)
        self.head = Linear(spec.hidden_size, spec.vocab_size)
        self.embed_post, self.logits_post = _stream_ops(spec)
        self.embed: torch.Tensor | None = None
        self.run = [RunEntry(e.layer, i if e.cache is None else e.cache) for i, e in enumerate(spec.run)]
        for i, e in enumerate(self.run):
            if not (0 <= e.layer < len(self.blocks)):
                raise ValueError(f"run entry {i} names layer {e.layer}, but the model has {len(self.blocks)} layers")
            if not (0 <= e.cache <= i):
                raise ValueError(f"run entry {i} reads the cache of entry {e.cache}, which does not run before it")
            if self.run[e.cache].cache != e.cache:
                raise ValueError(f"run entry {i} reads the cache of entry {e.cache}, which has no cache of its own")

    # ---- weights -------------------------------------------------------------------------------
    def expected_tensors(self):
        return expected_tensors(self.spec, self.blocks)

    def load(self, loader) -> None:
        exp, optional = self.expected_tensors()
        loader.check(exp, optional)
        self._load_from(lambda name, compute=False: loader.fetch(name, compute=compute), loader.has)

    def load_random(self, seed: int, device, dtype: torch.dtype) -> None:
        """Draws every tensor on the device by the rule of the random-weights mode (weights/random_init.py: each
        tensor from (seed, its name)); for measurements at sizes where writing a file first would only cost time."""
        from ..weights.random_init import draw_on_device
        exp, _ = self.expected_tensors()
        self._load_from(lambda name, compute=False: draw_on_device(seed, name, exp[name], dtype, device),
                        lambda name: name in exp)

    def _load_from(self, get, has) -> None:
        s = self.spec
        self.embed = get(s.embed_name, compute=True)
        for l, b in zip(s.layers, self.blocks):
            b.load(lambda n, _p=l.prefix, **kw: get(_p + n, **kw))
        self.final_norm.load(lambda n, **kw: get(s.final_norm_name + n, **kw))
        if has(s.head_name):
            self.head.set_weight(get(s.head_name, compute=True))
        elif s.tie_embeddings:
            self.head.set_weight(self.embed)  # one buffer for both
        else:
            raise ValueError(f"no {s.head_name} in the weights and tie_word_embeddings is false")
        for op in (self.embed_post, self.logits_post):
            if op is not None:
                op[1].load(lambda n, _p=op[0], **kw: get(_p + n, **kw))

    # ---- cache needs ---------------------------------------------------------------------------
    def cache_needs(self) -> list:
        """Per run entry: the CacheSpec of the cache it owns; None if it has none or borrows one."""
        out = []
        for i, e in enumerate(self.run):
            out.append(self.blocks[e.layer].mixer.cache_spec() if e.cache == i else None)
        return out

    def capturable(self) -> bool:
        """Whether a step of single rows may be captured once and replayed for other requests."""
        ops_ = [op[1] for op in (self.embed_post, self.logits_post) if op is not None]
        return (all(self.blocks[e.layer].capturable for e in self.run) and self.final_norm.capturable
                and all(o.capturable for o in ops_))

    def capturable_portions(self) -> bool:
        """The same for steps with prompt portions (Mixer.capturable_portions)."""
        return (self.capturable() and all(self.blocks[e.layer].capturable_portions for e in self.run)
                and self.final_norm.capturable_portions)

    # ---- execution -----------------------------------------------------------------------------
    def bind(self, ctx: BuildContext) -> None:
        self.ctx = ctx
        for b in self.blocks:
            b.bind(ctx)
        for op in (self.embed_post, self.logits_post):
            if op is not None:
                op[1].bind(ctx)
        ws = ctx.workspace
        self.hidden = ws.buffer("hidden", self.spec.hidden_size)
        self.final_normed = ws.buffer("final_normed", self.spec.hidden_size, rows=ctx.max_rows)
        self.logits = torch.empty((ctx.max_rows, self.spec.vocab_size), dtype=torch.float32, device=ctx.device)

    def forward(self, batch, caches: list) -> torch.Tensor:
        """Runs the batch's tokens through all run entries; returns float32 logits [num_rows, vocab]
        at batch.logits_rows (a view of a fixed buffer)."""
        T, R = batch.num_tokens, batch.num_rows
        ops.embedding(batch.input_ids[:T], self.embed, self.hidden, getattr(batch, "feedback_src", None),
                      getattr(batch, "last_tokens", None))
        if self.embed_post is not None:
            self.embed_post[1].forward(self.hidden, T)
        pending = None
        for i, e in enumerate(self.run):
            # the input norm of the block that runs next, if that block lets the one before carry it
            block = self.blocks[e.layer]
            if block.carries_norms and i + 1 < len(self.run):
                nxt = self.blocks[self.run[i + 1].layer].input_norm()
                pending = block.forward(self.hidden, pending, batch, caches[i], next_norm=nxt)
            else:
                pending = block.forward(self.hidden, pending, batch, caches[i])
        if R == 0:
            return self.logits[:0]
        if pending is None or isinstance(pending, Carried):
            self.final_norm.forward(self.hidden, self.final_normed, R, rows=batch.logits_rows)
        else:
            # the last add happens on the wanted rows only, inside the norm kernel
            self.final_norm.forward(pending, self.final_normed, R, residual=self.hidden, rows=batch.logits_rows)
        gemm.matmul_nt(self.final_normed, self.head.weight, self.logits, R, may_pad=True)  # both are buffers of max_rows rows
        if self.logits_post is not None:
            self.logits_post[1].forward(self.logits, R)
        return self.logits[:R]
