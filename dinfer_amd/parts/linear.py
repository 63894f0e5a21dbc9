"""y = x . W^T, W stored [out, in] row-major, no bias (crates/layers/src/nn.rs:16-76)."""
from __future__ import annotations

import torch

from ..kernels import gemm
from .base import Carried, Into


class Linear:
    def __init__(self, in_features: int, out_features: int):
        self.in_features, self.out_features = in_features, out_features
        self.weight: torch.Tensor | None = None

    def set_weight(self, w: torch.Tensor) -> None:
        if tuple(w.shape) != (self.out_features, self.in_features):
            raise ValueError(f"linear weight is {tuple(w.shape)}, expected {(self.out_features, self.in_features)}")
        self.weight = w.contiguous()

    def forward(self, x, out: torch.Tensor, m: int, scratch: bool = False) -> torch.Tensor:
        """scratch: x and out are activation buffers with spare rows beyond m that nothing reads. x may be a
        Carried: the norm it stands for is applied inside the product where a kernel does that."""
        if isinstance(x, Carried):
            if x.scaled and gemm.scaled_nt(x.xg, x.stats, x.cols, x.eps, x.width, self.weight, out, m):
                return out
            x = x.materialise()
        return gemm.matmul_nt(x, self.weight, out, m, may_pad=scratch)

    def forward_into(self, x: torch.Tensor, into: Into, m: int) -> Carried | None:
        """into.stream[:m] += x[:m] @ W^T, returning the Carried for into.norm; None (nothing done) where no kernel
        does this for the sizes. In steps of few rows the norm rides along (where it can be carried); a product of 17 to
        64 rows whose slices meet in a kernel of their own has that kernel write the norm's output as well (a Carried
        that is `ready`); in steps of many rows the product only adds, and the norm's kernel reads one matrix instead
        of two and writes one instead of two."""
        if into is None or into.norm is None or isinstance(x, Carried):
            return None
        width = self.out_features
        params = into.norm.carried()
        if params is not None and params[0] is not None and m <= into.xg.shape[0]:
            gain, offset, eps = params
            cols = gemm.sink_nt(x, self.weight, into.stream, into.xg, gain, offset, into.stats, m)
            if cols:
                return Carried(into.xg, into.stats, cols, eps, width, into.norm, into.stream, into.buf, m)
        if params is not None and params[0] is not None and gemm.mid_sink_nt(x, self.weight, into.stream, params[0],
                                                                            params[1], params[2], into.buf, m):
            return Carried(None, None, 0, 0.0, width, into.norm, into.stream, into.buf, m, ready=True)
        if gemm.add_nt(x, self.weight, into.stream, m):
            return Carried(None, None, 0, 0.0, width, into.norm, into.stream, into.buf, m)
        return None
