"""Matrix products out = a . w^T.

float32 operands: the vector-ALU kernel with a fixed summation order (the true
32-bit path). bfloat16 operands: up to 16 rows the hand-written MFMA kernel that
streams the weight once (decode, LM head); from 65 rows the vendor library, where
the reference uses a library too (crates/kernels/src/gemm.rs:605-647): hipBLASLt
called directly with the algorithm measured per shape (blaslt.py), or through
torch.mm where that library cannot be loaded. Between them (17 to 64 rows: decode
at larger batches) three kernels compete, and which wins depends on the weight's
shape: the few-row kernel, the kernel that keeps a slice of the activations in
LDS (csrc/gemm_mid.hip), and the library. They are timed once per shape, on the
operands of the first call, and the winner is kept.
"""
from __future__ import annotations

import os
import sys

import torch

from . import blaslt, ops

# Up to this many rows the weight-streaming kernel has no rival on MI355X (measured at the four layer shapes of an
# 8B model: one token tile, so the activations cost it a fraction of the weight's loads).
SMALL_M = 16
# Up to this many rows the hand-written kernels are candidates at all.
MID_M = 64
# (k per slice, row tiles per wave) of the LDS-resident kernel that are timed; what LDS does not hold is skipped
MID_FORMS = ((1024, 1), (1024, 2), (1536, 1), (2048, 1))

# Rows of a library product are rounded up to a multiple of this where the caller allows it: a prompt portion
# beside a changing number of decoding requests then meets a handful of shapes, each with its algorithm chosen
# once, instead of a new shape every step.
ROW_BUCKET = 32

_choice: dict = {}      # (device, row tiles, n, k, gated, out dtype, strides, may_pad) -> index into the candidate list
_workspace: dict = {}   # device -> float32 buffer for partial sums
_side: dict = {}        # device -> the stream candidates are captured on


def _tuning() -> bool:
    return os.environ.get("DINFER_GEMM_TUNE", "1") != "0" and not torch.cuda.is_current_stream_capturing()


def _mid_workspace(dev, need: int) -> torch.Tensor | None:
    """The buffer for partial sums, grown to `need` bytes; None where it would have to grow under capture."""
    ws = _workspace.get(dev)
    if ws is None or ws.numel() * 4 < need:
        if torch.cuda.is_current_stream_capturing():
            return None
        ws = _workspace[dev] = torch.empty((need + 3) // 4, dtype=torch.float32, device=dev)
    return ws


def _library(a, w, out, m, may_pad):
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


def _fastest(key, candidates) -> int:
    """Index of the fastest of the callables (each the whole product). Each is captured into a HIP graph of its
    own and the replay is timed, as decode steps run them: timed eagerly, a candidate pays for its host-side launch
    path too (tens of microseconds for a library call), which no step inside a graph ever sees. Before each of
    three replays a write empties the memory-side cache (in a model the weight comes from HBM); the least counts.
    A candidate that refuses the shape is skipped."""
    got = _choice.get(key)
    if got is not None:
        return got
    if not _tuning():
        return 0
    dev = key[0]
    flush = blaslt.flush_buffer(dev)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    side = _side.get(dev)
    if side is None:
        side = _side[dev] = torch.cuda.Stream(device=dev)
    best, best_t = 0, float("inf")
    times = {}
    for i, run in enumerate(candidates):
        if run is None:
            continue
        try:
            run()   # first use, eagerly: loads the kernel, lets the library choose its algorithm
            graph = torch.cuda.CUDAGraph()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                graph.capture_begin()
                try:
                    run()
                finally:
                    graph.capture_end()
            torch.cuda.current_stream().wait_stream(side)
            t = float("inf")
            for _ in range(3):
                flush.zero_()
                start.record()
                graph.replay()
                end.record()
                end.synchronize()
                t = min(t, start.elapsed_time(end))
            del graph
        except (RuntimeError, AssertionError):
            continue
        times[i] = round(t * 1e3, 1)
        if t < best_t:
            best, best_t = i, t
    _choice[key] = best
    if os.environ.get("DINFER_GEMM_TUNE_LOG"):
        print(f"[dinfer_amd] product {key[1:6]}: candidate {best} of {times} (us)", file=sys.stderr, flush=True)
    return best


def _mid_forms(a, w, out, m, gated):
    """The LDS-resident kernel in each of its forms, as callables; None for a form these sizes do not allow."""
    n = w.shape[0] // 2 if gated else w.shape[0]
    k = w.shape[1]
    runs = []
    for ks, rt in MID_FORMS:
        try:
            ws = _mid_workspace(a.device, ops.gemm_mid_m_workspace(m, n, k, gated=gated, ks=ks, rt=rt))
        except RuntimeError:
            ws = None
        runs.append(None if ws is None else
                    lambda ks=ks, rt=rt, ws=ws: ops.gemm_mid_m(a, w, out, m, ws, gated=gated, ks=ks, rt=rt))
    return runs


def matmul_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, may_pad: bool = False) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T; out has a's dtype, or float32 (logits). may_pad: a and out are scratch
    buffers whose rows beyond m hold nothing of value; the product may read and write a few of them."""
    if m <= 0:
        return out
    if a.dtype == torch.float32:
        return ops.gemm_ref(a, w, out, m)
    if not a.is_cuda:
        raise RuntimeError("matrix products run on the GPU only")
    n, k = w.shape
    if k % 8 or m > MID_M:
        return _library(a, w, out, m, may_pad)
    if m <= SMALL_M:
        return ops.gemm_small_m(a, w, out, m)
    # the first is what runs where nothing is measured: the few-row kernel up to 32 rows, the library beyond
    candidates = [lambda: ops.gemm_small_m(a, w, out, m) if m <= 32 else _library(a, w, out, m, may_pad),
                  lambda: _library(a, w, out, m, may_pad)]
    if m > 32:
        candidates.append(lambda: ops.gemm_small_m(a, w, out, m))
    candidates += _mid_forms(a, w, out, m, False) if n % 4 == 0 else [None] * len(MID_FORMS)
    key = (a.device, (m + 15) // 16, n, k, False, out.dtype, a.stride(0), out.stride(0), may_pad)
    (candidates[_fastest(key, candidates)] or candidates[0])()
    return out


def gated_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor, m: int, act: str) -> torch.Tensor:
    """out[:m] = act(a @ wg.T) * (a @ wu.T) for w = [wg; wu] stacked [2N, K]: the two projections of a gated
    feed-forward and its activation, in one kernel where one exists for the sizes. scratch [rows, 2N] takes the
    projections where the activation is a pass of its own."""
    if m <= 0:
        return out

    def two_passes():
        matmul_nt(a, w, scratch, m, may_pad=True)
        ops.gated_act(scratch, out, m, act)

    k = w.shape[1]
    if a.dtype != torch.bfloat16 or act != "silu" or k % 8 or m > MID_M:
        two_passes()
        return out
    if m <= SMALL_M:
        return ops.gemm_small_m_gated(a, w, out, m)
    candidates = [lambda: ops.gemm_small_m_gated(a, w, out, m) if m <= 32 else two_passes(), two_passes]
    candidates += _mid_forms(a, w, out, m, True) if out.shape[1] % 4 == 0 else [None] * len(MID_FORMS)
    key = (a.device, (m + 15) // 16, w.shape[0], k, True, out.dtype, a.stride(0), out.stride(0), True)
    (candidates[_fastest(key, candidates)] or candidates[0])()
    return out
