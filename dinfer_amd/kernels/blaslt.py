"""bf16 matrix products of many rows through hipBLASLt, the algorithm chosen per shape by measurement.

The reference hands these products to its vendor library too (crates/kernels/src/gemm.rs:605-647).
torch.mm asks hipBLASLt for its first suggestion; for few output tiles and a long K that suggestion is
far off (N 5,120, K 17,408 at 520 rows: 167 us against 102 us for the best of the library's own list),
so here the library is called directly: its candidate list for a shape is timed once, on the operands of
the first call, and the winner is kept for every later call of that shape.

out[M, N] = a[M, K] . w[N, K]^T in row-major storage is, in the library's column-major terms,
D (N x M, ld = ldc) = op_T(w as K x N, ld = ldw) . (a as K x M, ld = lda).
"""
from __future__ import annotations

import ctypes
import os
import sys
from ctypes import POINTER, byref, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

import torch

WORKSPACE_BYTES = 128 << 20   # for the library's split-K and stream-K kernels
CANDIDATES = 32               # how many of the library's suggestions are timed (the best has been seen as far down as 21st)
FLUSH_BYTES = 512 << 20       # read before each timed run: twice the memory-side cache
TUNE_FROM_ROWS = 33           # every size that comes here (up to 32 rows the weight-streaming kernel runs)
TUNE_FROM_WORK = 1 << 24      # rows x columns x depth below which no choice of kernel repays its measurement

_HIP_R_32F, _HIP_R_16BF = 0, 14
_OP_N, _OP_T = 111, 112
_COMPUTE_32F = 2
_DESC_TRANSA, _DESC_TRANSB = 0, 1
_PREF_MAX_WORKSPACE = 1


class _Algo(ctypes.Structure):
    _fields_ = [("data", ctypes.c_uint8 * 16), ("max_workspace_bytes", c_size_t)]


class _Heuristic(ctypes.Structure):
    _fields_ = [("algo", _Algo), ("workspace_size", c_size_t), ("state", c_int), ("waves_count", c_float),
                ("reserved", c_int * 4)]


_lib = None
_lib_tried = False
_handles: dict = {}
_workspaces: dict = {}
_plans: dict = {}
_flush: dict = {}
_one, _zero = c_float(1.0), c_float(0.0)


def _load():
    global _lib, _lib_tried
    if _lib_tried:
        return _lib
    _lib_tried = True
    if os.environ.get("DINFER_BLASLT", "1") == "0":
        return None
    # the copy torch itself has loaded comes first: one instance of the library and of its kernels per process
    for path in (os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so"),
                 "/opt/rocm/lib/libhipblaslt.so"):
        if os.path.exists(path):
            try:
                lib = ctypes.CDLL(path)
            except OSError:
                continue
            P = c_void_p
            lib.hipblasLtCreate.argtypes = [POINTER(P)]
            lib.hipblasLtMatmulDescCreate.argtypes = [POINTER(P), c_int, c_int]
            lib.hipblasLtMatmulDescSetAttribute.argtypes = [P, c_int, P, c_size_t]
            lib.hipblasLtMatrixLayoutCreate.argtypes = [POINTER(P), c_int, c_uint64, c_uint64, c_int64]
            lib.hipblasLtMatmulPreferenceCreate.argtypes = [POINTER(P)]
            lib.hipblasLtMatmulPreferenceSetAttribute.argtypes = [P, c_int, P, c_size_t]
            lib.hipblasLtMatmulPreferenceDestroy.argtypes = [P]
            lib.hipblasLtMatmulAlgoGetHeuristic.argtypes = [P, P, P, P, P, P, P, c_int, POINTER(_Heuristic),
                                                            POINTER(c_int)]
            lib.hipblasLtMatmul.argtypes = [P, P, P, P, P, P, P, P, P, P, P, P, POINTER(_Algo), P, c_size_t, P]
            _lib = lib
            break
    return _lib


def available() -> bool:
    return _load() is not None and ctypes.sizeof(_Heuristic) == 56


def _ok(status: int, what: str) -> None:
    if status != 0:
        raise RuntimeError(f"hipBLASLt {what} failed with status {status}")


class _Plan:
    """Descriptors of one problem shape and the algorithm that runs it."""
    __slots__ = ("desc", "lw", "la", "lc", "candidates", "algo", "tuned")

    def __init__(self, handle, m, n, k, lda, ldw, ldc, out_dtype):
        lib = _lib
        P = c_void_p
        self.desc, self.lw, self.la, self.lc = P(), P(), P(), P()
        _ok(lib.hipblasLtMatmulDescCreate(byref(self.desc), _COMPUTE_32F, _HIP_R_32F), "descriptor")
        for attr, op in ((_DESC_TRANSA, _OP_T), (_DESC_TRANSB, _OP_N)):
            v = c_int32(op)
            _ok(lib.hipblasLtMatmulDescSetAttribute(self.desc, attr, byref(v), 4), "descriptor attribute")
        ctype = _HIP_R_32F if out_dtype == torch.float32 else _HIP_R_16BF
        _ok(lib.hipblasLtMatrixLayoutCreate(byref(self.lw), _HIP_R_16BF, k, n, ldw), "layout")
        _ok(lib.hipblasLtMatrixLayoutCreate(byref(self.la), _HIP_R_16BF, k, m, lda), "layout")
        _ok(lib.hipblasLtMatrixLayoutCreate(byref(self.lc), ctype, n, m, ldc), "layout")
        pref = P()
        _ok(lib.hipblasLtMatmulPreferenceCreate(byref(pref)), "preference")
        ws = c_uint64(WORKSPACE_BYTES)
        _ok(lib.hipblasLtMatmulPreferenceSetAttribute(pref, _PREF_MAX_WORKSPACE, byref(ws), 8), "preference attribute")
        res = (_Heuristic * CANDIDATES)()
        got = c_int(0)
        _ok(lib.hipblasLtMatmulAlgoGetHeuristic(handle, self.desc, self.lw, self.la, self.lc, self.lc, pref, CANDIDATES,
                                                res, byref(got)), "heuristic")
        lib.hipblasLtMatmulPreferenceDestroy(pref)
        self.candidates = [res[i].algo for i in range(got.value)
                           if res[i].state == 0 and res[i].workspace_size <= WORKSPACE_BYTES]
        if not self.candidates:
            raise RuntimeError(f"hipBLASLt has no kernel for a {m} x {n} x {k} bf16 product")
        self.algo = self.candidates[0]
        self.tuned = False


def _run(handle, plan, algo, a, w, out, workspace, beta=_zero) -> None:
    """out = a . w^T + beta * out (the library reads and writes the same matrix)."""
    stream = torch.cuda.current_stream(a.device).cuda_stream
    _ok(_lib.hipblasLtMatmul(handle, plan.desc, byref(_one), w.data_ptr(), plan.lw, a.data_ptr(), plan.la, byref(beta),
                             out.data_ptr(), plan.lc, out.data_ptr(), plan.lc, byref(algo), workspace.data_ptr(),
                             WORKSPACE_BYTES, stream), "matmul")


def flush_caches(dev) -> None:
    """Reads FLUSH_BYTES of other memory, so that what runs next finds its operands in HBM, as a weight is found
    in a model whose other layers have passed through the caches since. Read, not written: lines written here
    would still be on their way out while the timed kernel runs, and compete with it."""
    flush = _flush.get(dev)
    if flush is None:
        flush = _flush[dev] = torch.zeros(FLUSH_BYTES // 4, dtype=torch.float32, device=dev)   # summed as it is: no widened copy
    flush.sum()


def _tune(handle, plan, a, w, out, workspace, beta=_zero) -> None:
    """Times every candidate on the call's own operands and keeps the fastest. In a model the weight of a
    product comes from HBM (the layers before have pushed it out of every cache), so each timed run follows a
    read of FLUSH_BYTES of other memory that empties the memory-side cache; timed on a weight that stays cached, kernels win
    that lose in place. A product that adds to its output is timed on a copy of it."""
    if beta is not _zero:
        out = out.clone()
    best, best_t, best_i, times = plan.candidates[0], float("inf"), 0, []
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i, algo in enumerate(plan.candidates):
        try:
            _run(handle, plan, algo, a, w, out, workspace, beta)   # first use of a kernel loads it
            t = float("inf")
            for _ in range(3):   # the least of three: a single timing wanders by a few per cent, as much as the candidates differ
                flush_caches(a.device)
                start.record()
                _run(handle, plan, algo, a, w, out, workspace, beta)
                end.record()
                end.synchronize()
                t = min(t, start.elapsed_time(end))
        except RuntimeError:
            continue
        times.append(round(t * 1e3, 1))
        if t < best_t:
            best, best_t, best_i = algo, t, i
    plan.algo, plan.tuned = best, True
    if os.environ.get("DINFER_GEMM_TUNE_LOG"):
        print(f"[dinfer_amd] library product {tuple(out.shape)[1]} x {tuple(a.shape)[1]}, {out.dtype}: algorithm {best_i} of {times} (us)",
              file=sys.stderr, flush=True)


def matmul(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, accumulate: bool = False) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T; a, w bfloat16 with contiguous rows, out bfloat16 or float32. accumulate: out[:m] +=
    instead, the sum of the float accumulators and out rounded once."""
    beta = _one if accumulate else _zero
    dev = a.device
    handle = _handles.get(dev)
    if handle is None:
        handle = c_void_p()
        with torch.cuda.device(dev):
            _ok(_lib.hipblasLtCreate(byref(handle)), "create")
            _workspaces[dev] = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=dev)
        _handles[dev] = handle
    n, k = w.shape
    key = (dev, m, n, k, a.stride(0), w.stride(0), out.stride(0), out.dtype, accumulate)
    plan = _plans.get(key)
    if plan is None:
        try:
            plan = _Plan(handle, m, n, k, a.stride(0), w.stride(0), out.stride(0), out.dtype)
        except RuntimeError:
            plan = False   # a shape the direct interface does not take: torch's own call of the library serves it
        _plans[key] = plan
    if plan is False:
        if accumulate:
            out[:m].addmm_(a[:m].to(out.dtype), w.t().to(out.dtype))
        elif out.dtype == a.dtype:
            torch.mm(a[:m], w.t(), out=out[:m])
        else:
            out[:m].copy_(torch.mm(a[:m], w.t()))
        return out
    workspace = _workspaces[dev]
    if (not plan.tuned and m >= TUNE_FROM_ROWS and m * n * k >= TUNE_FROM_WORK and len(plan.candidates) > 1
            and os.environ.get("DINFER_GEMM_TUNE", "1") != "0" and not torch.cuda.is_current_stream_capturing()):
        _tune(handle, plan, a, w, out, workspace, beta)
    _run(handle, plan, plan.algo, a, w, out, workspace, beta)
    return out
