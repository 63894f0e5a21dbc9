"""y = x . W^T, W stored [out, in] row-major, no bias (crates/layers/src/nn.rs:16-76)."""
from __future__ import annotations

import torch

from ..kernels import gemm


class Linear:
    def __init__(self, in_features: int, out_features: int):
        self.in_features, self.out_features = in_features, out_features
        self.weight: torch.Tensor | None = None

    def set_weight(self, w: torch.Tensor) -> None:
        if tuple(w.shape) != (self.out_features, self.in_features):
            raise ValueError(f"linear weight is {tuple(w.shape)}, expected {(self.out_features, self.in_features)}")
        self.weight = w.contiguous()

    def forward(self, x: torch.Tensor, out: torch.Tensor, m: int, scratch: bool = False) -> torch.Tensor:
        """scratch: x and out are activation buffers with spare rows beyond m that nothing reads."""
        return gemm.matmul_nt(x, self.weight, out, m, may_pad=scratch)
