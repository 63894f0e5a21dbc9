"""Gated feed-forward: down( act(gate(x)) * up(x) ), gate and up fused into one
[2I, hidden] operand with the gate rows first (crates/layers/src/nn.rs:272-390)."""
from __future__ import annotations

import torch

from ..kernels import gemm
from .base import FeedForward
from .linear import Linear
from .registry import FEED_FORWARDS
from .spec import TensorSpec


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, hidden: int, intermediate: int, act: str = "silu"):
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

    def forward(self, x, batch):
        T = batch.num_tokens
        # decode-sized steps: both projections and the activation in one weight-streaming kernel
        gemm.gated_nt(x, self.gate_up.weight, self.act_buf, self.gu_buf, T, self.act)
        return self.down.forward(self.act_buf, self.out_buf, T, scratch=True)
