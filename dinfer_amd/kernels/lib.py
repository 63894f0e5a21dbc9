"""Loads the compiled HIP libraries through ctypes and declares their C ABI.

There is no fallback: if a library is missing it is compiled; if that fails, or
no GPU is present when a kernel is called, the call raises.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_float, c_int, c_int64, c_uint32, c_void_p

from ..csrc import build as _build

_P = c_void_p
_I = c_int
_L = c_int64
_F = c_float

# function name -> (library, argument types). Every function returns an int status.
SIGNATURES = {
    "dinfer_embedding": ("elementwise", [_I, _P, _P, _P, _L, _L, _L, _P, _P, _P]),
    "dinfer_gated_act": ("elementwise", [_I, _I, _P, _P, _L, _L, _L, _P]),
    "dinfer_add_inplace": ("elementwise", [_I, _P, _P, _L, _P]),
    "dinfer_scale_softcap": ("elementwise", [_I, _P, _L, _L, _L, _F, _F, _P]),
    "dinfer_widen": ("elementwise", [_I, _P, _P, _L, _P]),
    "dinfer_fill_u32": ("elementwise", [_P, c_uint32, _L, _P]),
    "dinfer_rmsnorm": ("norm", [_I, _P, _P, _P, _P, _I, _P, _L, _L, _L, _L, _F, _F, _P]),
    "dinfer_qkv_post": (
        "rope",
        [_I, _P, _L, _L, _L, _L, _L, _P, _P, _I, _F, _F, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _P],
    ),
    "dinfer_attn_paged_ref": (
        "attention_ref",
        [_I, _P, _L, _P, _L, _P, _P, _P, _L, _P, _P, _I, _L, _F, _I, _I, _I, _I, _I, _P],
    ),
    "dinfer_attn_mfma_supports": ("attention", [_I, _I, _I, _I]),
    "dinfer_attn_flash": (
        "attention",
        [_P, _L, _P, _L, _P, _P, _P, _L, _P, _P, _I, _I, _F, _I, _I, _I, _I, _I, _I, _P],
    ),
    "dinfer_attn_decode": (
        "attention",
        [_P, _L, _P, _L, _P, _L, _P, _P, _P, _L, _P, _P, _I, _I, _F, _I, _I, _I, _I, _I, _P],
    ),
    "dinfer_attn_decode_post_supports": ("attention", [_I]),
    "dinfer_attn_decode_post": (
        "attention",
        [_P, _P, _P, _L, _P, _L, _P, _L, _P, _P, _P, _L, _P, _I, _I, _F, _I, _I, _I, _I, _I, _P, _P, _F, _F, _P, _P,
         _P, _P],
    ),
    "dinfer_gemm_ref": ("gemm_ref", [_I, _I, _P, _L, _P, _L, _P, _L, _L, _L, _L, _P]),
    "dinfer_gemm_small_m": ("gemm", [_I, _P, _L, _P, _L, _P, _L, _L, _L, _L, _I, _I, _P]),
    "dinfer_gemm_small_m_gated": ("gemm", [_P, _L, _P, _L, _P, _L, _L, _L, _L, _I, _P]),
    "dinfer_gemm_small_m_scaled": ("gemm", [_P, _L, _P, _L, _P, _L, _L, _L, _L, _I, _P, _L, _L, _F, _L, _P]),
    "dinfer_gemm_small_m_sink_stats_columns": ("gemm", [_L, _L, _L]),
    "dinfer_gemm_small_m_sink": ("gemm", [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _F, _P, _L, _L, _L, _L, _P]),
    "dinfer_gemm_mid_m": ("gemm_mid", [_I, _P, _L, _P, _L, _P, _L, _L, _L, _L, _I, _I, _I, _P, _L, _P]),
    "dinfer_gemm_mid_m_sink": ("gemm_mid", [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _F, _F, _L, _L, _L, _I, _I, _P, _L, _P]),
    "dinfer_gemm_mid_m_workspace": ("gemm_mid", [_L, _L, _L, _I, _I, _I, _P]),
    "dinfer_gemm_mid_m_static": ("gemm_mid", [_I, _P, _L, _P, _L, _P, _L, _L, _L, _L, _I, _I, _I, _P]),
    "dinfer_gemm_mid_m_static_init": ("gemm_mid", []),
    "dinfer_gemm_wide_supports": ("gemm_wide", [_L, _L, _L]),
    "dinfer_gemm_wide": ("gemm_wide", [_I, _P, _L, _P, _L, _P, _L, _L, _L, _L, _I, _P, _L, _I, _F, _L, _P]),
    "dinfer_stream_read": ("ceilings", [_P, _L, _I, _P, _P]),
    "dinfer_mfma_loop": ("ceilings", [_I, _I, _P, _P, _P]),
    "dinfer_argmax": ("sampling", [_P, _L, _P, _L, _L, _P, _L, _P]),
    "dinfer_argmax_scratch_bytes": ("sampling", [_L, _L, _P]),
    "dinfer_sample": ("sampling", [_P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _P]),
    "dinfer_sample_rows": ("sampling", [_P, _L, _P, _P, _L, _P, _P, _L, _L, _I, _I, _P]),
    "dinfer_sample_scratch_bytes": ("sampling", [_L, _L, _P]),
    "dinfer_history_add": ("sampling", [_P, _L, _L, _P, _L, _P]),
    "dinfer_penalties_dense": ("sampling", [_P, _L, _P, _L, _P, _L, _L, _P]),
    "dinfer_logit_bias": ("sampling", [_P, _L, _P, _P, _L, _L, _L, _P]),
    "dinfer_logprobs": ("sampling", [_P, _L, _P, _P, _L, _P, _P, _P, _L, _L, _P]),
}

ERRORS = {
    1: "unsupported dtype code",
    2: "operand shapes or strides do not fit the kernel",
    3: "size or option not supported by this kernel",
    4: "kernel launch failed",
    5: "workspace too small",
    6: "sizes beyond what the library's built-in scratch array holds",
}

_libs: dict[str, ctypes.CDLL] = {}
_funcs: dict[str, ctypes._CFuncPtr] = {}
_lock = threading.Lock()


class KernelError(RuntimeError):
    pass


def load_library(name: str) -> ctypes.CDLL:
    with _lock:
        lib = _libs.get(name)
        if lib is not None:
            return lib
        # only a library whose recorded hash equals the hash of today's sources is loaded: the argument lists
        # above belong to those sources, and a kernel launched through another list reads past its operands
        path = _build.find_built(name)
        if path is None:
            try:
                path = _build.build(name)
            except (RuntimeError, OSError) as e:
                raise KernelError(f"libdinfer_{name}.so is missing or older than its source and cannot be "
                                  f"built here: {e}") from e
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from e
        _libs[name] = lib
        return lib


def register(name: str, library: str, argtypes: list) -> None:
    """Declares a further entry point (used by libraries added later)."""
    SIGNATURES[name] = (library, argtypes)


def get(name: str):
    fn = _funcs.get(name)
    if fn is None:
        libname, argtypes = SIGNATURES[name]
        fn = getattr(load_library(libname), name)
        fn.argtypes = argtypes
        fn.restype = c_int
        _funcs[name] = fn
    return fn


def call(name: str, *args) -> None:
    rc = get(name)(*args)
    if rc != 0:
        raise KernelError(f"{name}: {ERRORS.get(rc, f'status {rc}')}")


def loaded_libraries() -> list[str]:
    return sorted(_libs)
