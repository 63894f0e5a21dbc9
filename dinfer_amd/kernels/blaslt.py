"""bf16 matrix products of many rows through hipBLASLt, the algorithm chosen per shape by measurement.

The reference hands these products to its vendor library too (crates/kernels/src/gemm.rs:605-647).
The library's first suggestion is what a framework's own matmul runs; for few output tiles and a long K it is
far off (N 5,120, K 17,408 at 520 rows: 167 us against 102 us for the best of the library's own list),
so here the library is called directly and its candidate list for a shape is timed.

When it is timed, and what a product runs with otherwise, is settled so that results repeat:
  * a product outside `measuring()` never times anything: it runs the algorithm its shape was given earlier,
    or the library's first suggestion. The engine's warm-up runs one step of every row count under
    `measuring()`, before it serves; no serving step stalls for a measurement.
  * of the timed candidates the one with the lowest index within TIE of the fastest wins, so two runs that
    time the same candidates a per cent apart choose the same one.
  * the choices are kept in a plan file beside the built libraries, keyed by device, library and shape; a later
    process finds them there, measures nothing and computes the same bits as the one that measured.
  * `configure(tuning="heuristic")` takes the library's first suggestion everywhere (no measurement, no file).
These are engine options (EngineOptions.gemm_tuning, gemm_plan_file), not environment switches. A shape the
library names no algorithm for is left to the caller (`matmul` returns False), who runs the plain kernel.

out[M, N] = a[M, K] . w[N, K]^T in row-major storage is, in the library's column-major terms,
D (N x M, ld = ldc) = op_T(w as K x N, ld = ldw) . (a as K x M, ld = lda).
"""
from __future__ import annotations

import contextlib
import ctypes
import json
import os
import sys
from ctypes import POINTER, byref, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

import torch

WORKSPACE_BYTES = 128 << 20   # for the library's split-K and stream-K kernels
CANDIDATES = 32               # how many of the library's suggestions are timed (the best has been seen as far down as 21st)
FLUSH_BYTES = 512 << 20       # read before each timed run: twice the memory-side cache
TUNE_FROM_ROWS = 33           # every size that comes here (up to 32 rows the weight-streaming kernel runs)
TUNE_FROM_WORK = 1 << 24      # rows x columns x depth below which no choice of kernel repays its measurement
TIE = 0.03                    # candidates within this fraction of the fastest count as equal: the lowest index wins

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

# settings of the process (the engine sets them from its options when it is built)
_settings = {"tuning": "measured", "plan_file": None, "log": False}
_measuring = False            # inside measuring(): shapes without a choice are timed
_stored: dict | None = None   # the plan file's contents: shape key -> {"index": i, "algo": hex of the algorithm's bytes}
_stored_path = None


def configure(tuning: str | None = None, plan_file=..., log: bool | None = None) -> None:
    """tuning "measured": candidates are timed inside measuring() and the choices kept in the plan file;
    "heuristic": the library's first suggestion for every shape. plan_file: where choices are kept between
    processes ("" for nowhere; None: beside the built libraries; left out: as it was). Arguments left out or None
    (plan_file aside) change nothing. Shapes that already have a plan keep it."""
    global _stored, _stored_path
    if tuning is not None and tuning not in ("measured", "heuristic"):
        raise ValueError(f"gemm tuning must be 'measured' or 'heuristic', got {tuning!r}")
    for k, v in (("tuning", tuning), ("log", log)):
        if v is not None:
            _settings[k] = v
    if plan_file is not ... and plan_file != _settings["plan_file"]:
        _save_stored()
        _settings["plan_file"] = plan_file
        _stored = _stored_path = None


@contextlib.contextmanager
def measuring():
    """Products of shapes that have no choice yet time their candidates in here (the engine's warm-up)."""
    global _measuring
    before, _measuring = _measuring, _settings["tuning"] == "measured"
    try:
        yield
    finally:
        _measuring = before
        _save_stored()


def _plan_path(dev):
    global _stored_path
    if _stored_path is None:
        f = _settings["plan_file"]
        if f == "":
            return None
        if f is None:
            from ..csrc import build
            import hashlib
            ident = f"{torch.cuda.get_device_name(dev)}|{torch.version.hip}|{CANDIDATES}|{WORKSPACE_BYTES}"
            f = str(build.lib_dir() / f"blaslt_plans_{hashlib.sha256(ident.encode()).hexdigest()[:12]}.json")
        _stored_path = f
    return _stored_path


_stored_dirty = False
worth_measuring_met = 0       # how many products so far were of a size whose algorithm is worth measuring


def _load_stored(dev) -> dict:
    global _stored
    if _stored is None:
        _stored = {}
        path = _plan_path(dev)
        if path and os.path.exists(path):
            try:
                with open(path) as fh:
                    data = json.load(fh)
                if isinstance(data, dict):
                    _stored = data
            except (OSError, ValueError):
                pass   # an unreadable file is measured again and rewritten
    return _stored


def _save_stored() -> None:
    global _stored_dirty
    if not _stored_dirty or _stored is None or not _stored_path:
        return
    _stored_dirty = False
    try:
        # other processes may have added shapes since this one read the file
        merged = {}
        if os.path.exists(_stored_path):
            try:
                with open(_stored_path) as fh:
                    merged = json.load(fh)
            except (OSError, ValueError):
                merged = {}
        merged.update(_stored)
        tmp = f"{_stored_path}.{os.getpid()}.tmp"
        with open(tmp, "w") as fh:
            json.dump(merged, fh, indent=0, sort_keys=True)
        os.replace(tmp, _stored_path)
    except OSError:
        pass   # a folder that cannot be written: the choices live as long as the process


def _load():
    global _lib, _lib_tried
    if _lib_tried:
        return _lib
    _lib_tried = True
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


def require() -> None:
    if not available():
        raise RuntimeError("hipBLASLt cannot be loaded (looked beside torch's libraries and in /opt/rocm/lib): the "
                           "bfloat16 products of more than 32 rows have no other library")


def _ok(status: int, what: str) -> None:
    if status != 0:
        raise RuntimeError(f"hipBLASLt {what} failed with status {status}")


class _Plan:
    """Descriptors of one problem shape and the algorithm that runs it."""
    __slots__ = ("desc", "lw", "la", "lc", "candidates", "algo", "tuned", "index", "times", "asked")

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
        self.algo, self.index, self.times = self.candidates[0], 0, None
        self.tuned = False   # True once the choice was measured here or taken from the plan file
        self.asked = False   # True once the plan file was asked about this shape


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the handle alone: building a Stream object costs 4 us a call


def _run(handle, plan, algo, a, w, out, workspace, beta=_zero) -> None:
    """out = a . w^T + beta * out (the library reads and writes the same matrix)."""
    stream = _raw_stream(a.device.index) if _raw_stream is not None else torch.cuda.current_stream(a.device).cuda_stream
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
    times = []
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i, algo in enumerate(plan.candidates):
        t = float("inf")
        try:
            _run(handle, plan, algo, a, w, out, workspace, beta)   # first use of a kernel loads it
            for _ in range(3):   # the least of three: a single timing wanders by a few per cent, as much as the candidates differ
                flush_caches(a.device)
                start.record()
                _run(handle, plan, algo, a, w, out, workspace, beta)
                end.record()
                end.synchronize()
                t = min(t, start.elapsed_time(end))
        except RuntimeError:
            t = float("inf")
        times.append(t)
    fastest = min(times)
    # the first candidate within TIE of the fastest: two measurements a per cent apart choose the same one
    index = next(i for i, t in enumerate(times) if t <= fastest * (1.0 + TIE)) if fastest < float("inf") else 0
    plan.algo, plan.index, plan.tuned = plan.candidates[index], index, True
    plan.times = [round(t * 1e3, 1) if t < float("inf") else None for t in times]
    if _settings["log"]:
        print(f"[dinfer_amd] library product {tuple(out.shape)[1]} x {tuple(a.shape)[1]}, {out.dtype}: algorithm {index} of "
              f"{plan.times} (us)", file=sys.stderr, flush=True)


def _shape_key(m, n, k, lda, ldw, ldc, out_dtype, accumulate) -> str:
    return f"{m},{n},{k},{lda},{ldw},{ldc},{'f32' if out_dtype == torch.float32 else 'bf16'},{int(accumulate)}"


def chosen() -> list:
    """What every shape met so far runs with: rows, columns, depth, index in the library's list, how it was chosen."""
    out = []
    for key, plan in _plans.items():
        if plan:
            _, m, n, k = key[:4]
            out.append({"m": m, "n": n, "k": k, "accumulate": bool(key[-1]), "algorithm": plan.index,
                        "chosen": "measured" if plan.tuned else "first suggestion"})
    return out


def matmul(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, accumulate: bool = False) -> bool:
    """out[:m] = a[:m] @ w.T; a, w bfloat16 with contiguous rows, out bfloat16 or float32. accumulate: out[:m] +=
    instead, the sum of the float accumulators and out rounded once. False, and nothing done, where the library has
    no algorithm for the shape."""
    require()
    if not (a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1):
        raise ValueError("library products take operands with contiguous rows")
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
            plan = False   # a shape the library takes no algorithm for
        _plans[key] = plan
    if plan is False:
        return False
    workspace = _workspaces[dev]
    if (not plan.tuned and _settings["tuning"] == "measured" and m >= TUNE_FROM_ROWS and m * n * k >= TUNE_FROM_WORK
            and len(plan.candidates) > 1):
        _choose(handle, plan, key, a, w, out, workspace, beta)
    _run(handle, plan, plan.algo, a, w, out, workspace, beta)
    return True


def _choose(handle, plan, key, a, w, out, workspace, beta) -> None:
    """Gives a shape its algorithm: from the plan file if it is there (and names a candidate the library still
    lists at that place), else, inside measuring(), by timing. Outside measuring() a shape without a stored choice
    keeps the library's first suggestion and stays open for a later warm-up."""
    global _stored_dirty, worth_measuring_met
    worth_measuring_met += 1
    if plan.asked and not _measuring:
        return
    dev = key[0]
    skey = _shape_key(*key[1:])
    stored = None if plan.asked else _load_stored(dev).get(skey)
    plan.asked = True
    if stored is not None:
        i = stored.get("index", -1)
        if 0 <= i < len(plan.candidates) and bytes(plan.candidates[i].data).hex() == stored.get("algo"):
            plan.algo, plan.index, plan.tuned = plan.candidates[i], i, True
            return
    if not _measuring or torch.cuda.is_current_stream_capturing():
        return
    _tune(handle, plan, a, w, out, workspace, beta)
    _stored[skey] = {"index": plan.index, "algo": bytes(plan.candidates[plan.index].data).hex()}
    _stored_dirty = True
