"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * (w + offset), float arithmetic
(crates/layers/src/nn.rs:78-111, crates/kernels/cuda/rmsnorm_core.cuh:63-81)."""
from __future__ import annotations

from ..kernels import ops
from .base import Norm
from .registry import NORMS
from .spec import TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, width: int, eps: float, weight_offset: float = 0.0):
        self.width, self.eps, self.weight_offset = width, eps, weight_offset
        self.weight = None

    def tensors(self):
        return {"weight": TensorSpec((self.width,), init="gain")}

    def load(self, get):
        self.weight = get("weight")

    def carried(self):
        return (self.weight, self.weight_offset, self.eps)

    def forward(self, x, out, n_rows, *, residual=None, rows=None):
        return ops.rmsnorm(x, self.weight, out, self.eps, n_rows, residual=residual, rows=rows,
                           weight_offset=self.weight_offset)
