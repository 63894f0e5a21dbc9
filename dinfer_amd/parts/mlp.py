"""Gated feed-forward: down( act(gate(x)) * up(x) ), gate and up fused into one
[2I, hidden] operand with the gate rows first (crates/layers/src/nn.rs:272-390)."""
from __future__ import annotations

import torch

from ..kernels import gemm, ops
from .base import Carried, FeedForward
from .linear import Linear
from .registry import FEED_FORWARDS
from .spec import TensorSpec


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(FeedForward):
    carries_norms = True   # the gate/up product takes a Carried, the down product an Into

    def __init__(self, hidden: int, intermediate: int, act: str = "silu"):
        if act not in ops.GATED_ACTS:   # said when the model is built, not at its first step
            raise ValueError(f"gated feed-forward: activation {act!r} has no kernel (known: {sorted(ops.GATED_ACTS)})")
        self.hidden, self.intermediate, self.act = hidden, intermediate, act
        self.gate_up = Linear(hidden, 2 * intermediate)
        self.down = Linear(intermediate, hidden)

    def tensors(self):
        return {
            "gate_proj.weight": TensorSpec((self.intermediate, self.hidden)),
            "up_proj.weight": TensorSpec((self.intermediate, self.hidden)),
            "down_proj.weight": TensorSpec((self.hidden, self.intermediate)),
        }

    def load(self, get):
        self.gate_up.set_weight(torch.cat([get("gate_proj.weight", compute=True),
                                           get("up_proj.weight", compute=True)], dim=0))
        self.down.set_weight(get("down_proj.weight", compute=True))

    def bind(self, ctx):
        ws = ctx.workspace
        self.gu_buf = ws.buffer("gate_up", 2 * self.intermediate)
        self.act_buf = ws.buffer("act", self.intermediate)
        self.out_buf = ws.buffer("ffn_out", self.hidden)

    def forward(self, x, batch, into=None):
        T = batch.num_tokens
        w = self.gate_up.weight
        if isinstance(x, Carried):
            if not (x.scaled and self.act == "silu" and gemm.scaled_nt(x.xg, x.stats, x.cols, x.eps, x.width, w, self.act_buf, T, gated=True)):
                x = x.materialise()
        if not isinstance(x, Carried):
            # decode-sized steps: both projections and the activation in one weight-streaming kernel
            gemm.gated_nt(x, w, self.act_buf, self.gu_buf, T, self.act)
        if into is not None:
            done = self.down.forward_into(self.act_buf, into, T)
            if done is not None:
                return done
        return self.down.forward(self.act_buf, self.out_buf, T, scratch=True)
