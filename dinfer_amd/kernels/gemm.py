"""Matrix products out = a . w^T.

float32 operands: the vector-ALU kernel with a fixed summation order (the true
32-bit path). bfloat16 operands: up to 32 rows the hand-written MFMA kernel that
streams the weight once (decode, LM head); beyond, the vendor library, where the
reference uses a library too (crates/kernels/src/gemm.rs:605-647): hipBLASLt
called directly with the algorithm measured per shape (blaslt.py); a shape it
names no algorithm for runs the plain kernel. One shape is taken from both at 17
to 64 rows: a weight with far more columns than rows (the down projection of a
feed-forward), where the few-row kernel drowns in loads of the activations and
the library has few output tiles to spread; the kernel that keeps a slice of the
activations in LDS (csrc/gemm_mid.hip) runs it.

Which kernel runs is a rule of the sizes, not a measurement at run time. A
measurement was tried (every candidate captured into a graph of its own, timed
after the caches were emptied) and did not predict the order inside a decode
step: at 64 rows it chose the LDS kernel for the gate and up projections, which
timed 8 % ahead alone and cost 0.1 ms a step in place. The rule below is what whole
decode steps of an 8B-sized model measured.
"""
from __future__ import annotations

import torch

from . import blaslt, ops

# Up to this many rows the weight-streaming kernel beats the library on MI355X (measured at the four layer
# shapes of an 8B model and at a 152k vocabulary: ahead up to 32 rows, level at 48, behind at 64).
SMALL_M = 32
# Up to this many rows the LDS-resident kernel takes the weights that are at least TALL times as wide as high and
# at least TALL_BYTES large (below, a launch costs more than any kernel saves).
MID_M = 64
TALL = 2
TALL_BYTES = 32 << 20

# Rows of a library product are rounded up where the caller allows it: a prompt portion beside a changing number of
# decoding requests then meets a handful of shapes, each with its algorithm chosen once, instead of a new shape
# every step. Up to 1,024 rows to a multiple of 32; beyond, in coarser steps (at most an eighth more rows), so that
# the shapes an engine can meet stay a few dozen however large its step budget is.


def row_bucket(m: int) -> int:
    """The row count a product of m rows runs with where padding is allowed."""
    step = 32 if m <= 1024 else 128 if m <= 4096 else 512 if m <= 16384 else 2048
    return -(-m // step) * step


def row_buckets(most: int) -> list:
    """Every value row_bucket takes for 1 <= m <= most, ascending (the last may exceed `most`)."""
    out, m = [], 1
    while m <= most:
        b = row_bucket(m)
        out.append(b)
        m = b + 1
    return out

WIDE_CUS = 256          # the CUs the rule for csrc/gemm_wide.hip was measured on (MI355X)
_workspace: dict = {}   # device -> float32 buffer for partial sums
_outgrown: list = []    # earlier, smaller buffers: graphs captured with them still write there


def _mid_workspace(dev, need: int) -> torch.Tensor | None:
    """The buffer for partial sums, grown to `need` bytes; None where it would have to grow under capture.
    A buffer that is outgrown is kept, never freed: a captured graph holds its address."""
    ws = _workspace.get(dev)
    if ws is None or ws.numel() * 4 < need:
        if torch.cuda.is_current_stream_capturing():
            return None
        if ws is not None:
            _outgrown.append(ws)
            need = max(need, 2 * ws.numel() * 4)
        ws = _workspace[dev] = torch.empty((need + 3) // 4, dtype=torch.float32, device=dev)
    return ws


def _library(a, w, out, m, may_pad):
    # float32 out (logits at many positions): straight from the accumulators, as the few-row kernel gives them
    rows = min(a.shape[0], out.shape[0], row_bucket(m)) if may_pad else m
    if not blaslt.matmul(a, w, out, rows):
        ops.gemm_ref(a, w, out, m)      # a shape the library names no algorithm for: the plain kernel takes any
    return out


def _tall(m: int, n: int, k: int) -> bool:
    return 16 < m <= MID_M and k >= TALL * n and n % 4 == 0 and n * k * 2 >= TALL_BYTES


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
    if k % 8 == 0 and _tall(m, n, k):
        ks, rt = _mid_shape(m)
        ws = _mid_workspace(a.device, ops.gemm_mid_m_workspace(m, n, k, ks=ks, rt=rt))
        if ws is not None:
            return ops.gemm_mid_m(a, w, out, m, ws, ks=ks, rt=rt)
    if m <= SMALL_M and k % 8 == 0:
        return ops.gemm_small_m(a, w, out, m)
    return _library(a, w, out, m, may_pad)


def _mid_shape(m: int) -> tuple[int, int]:
    # slices of 1,536 with one row tile a wave where LDS holds them (up to 32 rows), else of 1,024 with two
    return (1536, 1) if m <= 32 else (1024, 2)


def mid_sink_nt(a: torch.Tensor, w: torch.Tensor, stream: torch.Tensor, gain: torch.Tensor, offset: float, eps: float,
                out: torch.Tensor, m: int) -> bool:
    """stream[:m] += a[:m] @ w.T in place and out[:m] = the RMSNorm (gain + offset, eps) of the new stream, for the
    products of 17 to 64 rows that the LDS-resident kernel takes (a weight far wider than high: the down projection):
    the pass over its partial sums is the add and the norm as well. False (nothing done) otherwise."""
    n, k = w.shape
    if not (a.is_cuda and a.dtype == torch.bfloat16 and stream.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
            and k % 8 == 0 and _tall(m, n, k) and n <= ops.GEMM_MID_SINK_MAX_N
            and gain.dtype in (torch.bfloat16, torch.float32)):
        return False
    ks, rt = _mid_shape(m)
    ws = _mid_workspace(a.device, ops.gemm_mid_m_workspace(m, n, k, ks=ks, rt=rt))
    if ws is None:
        return False
    ops.gemm_mid_m_sink(a, w, stream, out, gain, offset, eps, m, ws, ks=ks, rt=rt)
    return True


WIDE_FROM = 17   # up to 16 rows the few-row kernel is level with it (and carries norms)


def _wide(m: int, n: int, k: int) -> bool:
    """17 to 64 rows of a gated product go to the kernel whose waves stage their own activations (csrc/gemm_wide.hip)
    where its workgroups of 48 columns make one round over the CUs that is at least three quarters full. Measured
    with weights taken in turn, 12,288 columns of K = 4,096 (256 workgroups): against the few-row kernel 33.9 against
    35.2 us at 17 rows, 33.9 against 36.6 at 24, 34.8 against 38.7 at 32 (level at 8 and 16); against the library's
    product plus the activation kernel 37.1 against 51.1 us at 33 rows, 38.0 against 49.5 at 48, 42.6 against 49.6 at
    64. With a round and a half of workgroups (17,408 columns: 363) it loses to the library, 84 to 105 against 76 us,
    and with two it loses too."""
    groups = -(-n // 48)
    return WIDE_FROM <= m <= MID_M and WIDE_CUS * 3 // 4 < groups <= WIDE_CUS and ops.gemm_wide_supports(m, n, k)


def gated_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor, m: int, act: str) -> torch.Tensor:
    """out[:m] = act(a @ wg.T) * (a @ wu.T) for w = [wg; wu] stacked [2N, K]: the two projections of a gated
    feed-forward and its activation, in one weight-streaming kernel at decode sizes (up to 32 rows, up to 64 where
    the kernel for wide weights takes it). scratch
    [rows, 2N] takes the projections where the activation is a pass of its own."""
    if m <= 0:
        return out
    if a.dtype == torch.bfloat16 and act == "silu" and _wide(m, w.shape[0] // 2, w.shape[1]):
        return ops.gemm_wide(a, w, out, m, gated=True)
    if a.dtype == torch.bfloat16 and act == "silu" and m <= SMALL_M and w.shape[1] % 8 == 0:
        return ops.gemm_small_m_gated(a, w, out, m)
    matmul_nt(a, w, scratch, m, may_pad=True)
    ops.gated_act(scratch, out, m, act)
    return out


STATS_COLUMNS = 8   # a product that carries a norm leaves one sum of squares per token and this many columns, or twice as many
CARRY_M = 32   # the products that carry a norm take up to this many rows (the block arrangement asks for fewer)


def sink_nt(a: torch.Tensor, w: torch.Tensor, stream: torch.Tensor, xg: torch.Tensor, gain: torch.Tensor, offset: float,
            stats: torch.Tensor, m: int) -> int:
    """stream[:m] += a[:m] @ w.T in place, leaving xg = stream * (gain + offset) and per-row partial sums of squares in
    stats for the RMSNorm that reads the stream next: returns how many of them a row has. 0 (nothing done) where no
    kernel does this for the sizes."""
    n, k = w.shape
    if not (a.is_cuda and a.dtype == torch.bfloat16 and 0 < m <= CARRY_M and k % 8 == 0 and not _tall(m, n, k)):
        return 0
    return ops.gemm_small_m_sink(a, w, stream, xg, gain, stats, m, gain_offset=offset)


def add_nt(a: torch.Tensor, w: torch.Tensor, stream: torch.Tensor, m: int) -> bool:
    """stream[:m] += a[:m] @ w.T in place through the library (its `beta = 1`): the sum of the float accumulators and the
    stream, rounded once. For the steps of many rows, where sink_nt has no kernel; a and stream are activation buffers
    (rows beyond m hold nothing of value). False (nothing done) where the library does not run the product."""
    n, k = w.shape
    if not (a.is_cuda and a.dtype == torch.bfloat16 and stream.dtype == torch.bfloat16 and m > SMALL_M
            and not _tall(m, n, k)):
        return False
    rows = min(a.shape[0], stream.shape[0], row_bucket(m))
    return blaslt.matmul(a, w, stream, rows, accumulate=True)


def scaled_nt(xg: torch.Tensor, stats: torch.Tensor, cols: int, eps: float, width: int, w: torch.Tensor, out: torch.Tensor,
              m: int, gated: bool = False) -> bool:
    """out[:m] = (xg[:m] @ w.T) * rsqrt(sum(stats[r, :cols]) / width + eps), the product of the normed stream; gated: w is
    [gate; up] and out = silu(gate part) * up part. False (nothing done) where no kernel does this for the sizes."""
    n, k = (w.shape[0] // 2 if gated else w.shape[0]), w.shape[1]
    if not (xg.is_cuda and xg.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and 0 < m <= CARRY_M and k % 8 == 0
            and (gated or not _tall(m, n, k))):
        return False
    ops.gemm_small_m_scaled(xg, w, out, m, stats, cols, eps, width, gated=gated)
    return True
