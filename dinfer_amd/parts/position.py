"""Position encodings. The mixer's kernel rotates q and k by a table this part builds.

Rotary: row p of the table is [cos(p f_i) | sin(p f_i)], f_i = theta^(-2i / rotary_dim),
i < rotary_dim / 2, computed in float64 on the host and stored in float32
(crates/layers/src/nn.rs:152-185). rotary_dim may be smaller than the head
size (the other dims are not rotated); style selects the pairing.
"""
from __future__ import annotations

import torch

from .base import PositionEncoding
from .registry import POSITION_ENCODINGS

STYLES = {"neox": 0, "interleaved": 1}


@POSITION_ENCODINGS.register("none")
class NoPosition(PositionEncoding):
    def __init__(self, head_dim: int = 0, **_):
        self.rotary_dim, self.style = 0, 0

    def table(self):
        return None


@POSITION_ENCODINGS.register("rotary")
class Rotary(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, max_positions: int, rotary_dim: int | None = None,
                 style: str = "neox"):
        rd = head_dim if rotary_dim is None else rotary_dim
        if rd <= 0 or rd > head_dim or rd % 2:
            raise ValueError(f"rotary_dim {rd} must be even and in (0, head_dim={head_dim}]")
        if style not in STYLES:
            raise ValueError(f"rotary style {style!r} unknown; known: {sorted(STYLES)}")
        self.head_dim, self.theta, self.max_positions = head_dim, float(theta), max_positions
        self.rotary_dim, self.style = rd, STYLES[style]
        self._table = None

    def bind(self, ctx):
        # one table for all layers with the same rotation, as long as the longest request the engine admits
        n = min(self.max_positions, ctx.max_seq_len or self.max_positions)
        self._table = ctx.share(("rotary", self.theta, self.rotary_dim, self.style, n),
                                lambda: self.host_table(n).to(ctx.device).contiguous())

    def host_table(self, positions: int | None = None) -> torch.Tensor:
        i = torch.arange(0, self.rotary_dim // 2, dtype=torch.float64)
        freq = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / self.rotary_dim)
        ang = torch.arange(positions or self.max_positions, dtype=torch.float64)[:, None] * freq[None, :]
        return torch.cat([ang.cos(), ang.sin()], dim=1).to(torch.float32)

    def table(self):
        if self._table is None:
            raise RuntimeError("the rotation table is built in bind(); the part has not been bound")
        return self._table
