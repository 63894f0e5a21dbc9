"""Matrix products out = a . w^T.

float32 operands: the vector-ALU kernel with a fixed summation order (the true
32-bit path). bfloat16 operands: the hand-written MFMA kernel that streams the
weight once for few rows (decode, LM head), and the vendor library for many
rows, where the reference uses a library too (crates/kernels/src/gemm.rs:605-647):
hipBLASLt called directly with the algorithm measured per shape (blaslt.py), or
through torch.mm where that library cannot be loaded.
"""
from __future__ import annotations

import torch

from . import blaslt, ops


# Up to this many rows the weight-streaming kernel beats the library on MI355X (measured at the four layer
# shapes of an 8B model and at a 152k vocabulary: ahead up to 32 rows, level at 48, behind at 64).
SMALL_M = 32


def fuses_gated_act(a: torch.Tensor, w: torch.Tensor, m: int, act: str) -> bool:
    """Whether the gate/up projections and the activation of a gated feed-forward run as one kernel."""
    return a.dtype == torch.bfloat16 and act == "silu" and 0 < m <= SMALL_M and w.shape[1] % 8 == 0


# Rows of a library product are rounded up to a multiple of this where the caller allows it: a prompt portion
# beside a changing number of decoding requests then meets a handful of shapes, each with its algorithm chosen
# once, instead of a new shape every step.
ROW_BUCKET = 32


def matmul_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, may_pad: bool = False) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T; out has a's dtype, or float32 (logits). may_pad: a and out are scratch
    buffers whose rows beyond m hold nothing of value; the product may read and write a few of them."""
    if m <= 0:
        return out
    if a.dtype == torch.float32:
        return ops.gemm_ref(a, w, out, m)
    if not a.is_cuda:
        raise RuntimeError("matrix products run on the GPU only")
    if m <= SMALL_M and w.shape[1] % 8 == 0:
        return ops.gemm_small_m(a, w, out, m)
    if blaslt.available() and a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1:
        # float32 out (logits at many positions): straight from the accumulators, as the few-row kernel gives them
        rows = min(a.shape[0], out.shape[0], -(-m // ROW_BUCKET) * ROW_BUCKET) if may_pad else m
        return blaslt.matmul(a, w, out, rows)
    if out.dtype == torch.float32:
        tmp = torch.mm(a[:m], w.t())
        ops.widen(tmp, out, m * w.shape[0]) if out.is_contiguous() else out[:m].copy_(tmp)
        return out
    torch.mm(a[:m], w.t(), out=out[:m])
    return out
