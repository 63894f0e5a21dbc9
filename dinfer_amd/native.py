"""ctypes binding of the host core (csrc/host): page pools, cache manager, scheduler and
batch fill are C++; the classes in ``cache/`` and ``engine/`` are thin fronts over it.

A failing call returns minus the kind of its error; the text comes from dh_last_error().
"""
from __future__ import annotations

from ctypes import POINTER, Structure, c_char_p, c_int32, c_int64, c_void_p

from .kernels.lib import load_library

MAX_GROUPS = 8
_I, _L, _P = c_int32, c_int64, c_void_p
_PI, _PL = POINTER(c_int32), POINTER(c_int64)


class BatchBuffers(Structure):
    _fields_ = [("n_groups", _I), ("max_tokens", _I), ("max_reqs", _I), ("max_rows", _I),
                ("input_ids", _P), ("positions", _P), ("cu_seqlens", _P), ("seq_lens", _P),
                ("state_slots", _P), ("logits_rows", _P), ("feedback_src", _P),
                ("slot_mapping", _P * MAX_GROUPS), ("block_table", _P * MAX_GROUPS),
                ("max_blocks", _I * MAX_GROUPS)]


class BatchFacts(Structure):
    _fields_ = [(n, _I) for n in ("num_tokens", "num_reqs", "num_rows", "max_q_len", "max_seq_len", "num_singles")]


class SchedOptions(Structure):
    _fields_ = [(n, _I) for n in ("max_num_batched_tokens", "max_num_seqs", "max_model_len", "prefill_tokens_per_step",
                                  "long_prefill_token_threshold", "enable_chunked_prefill",
                                  "decode_exempt_from_budget", "enable_prefix_caching", "prefill_chunk_alignment",
                                  "max_logits_rows")]


class Scheduled(Structure):
    _fields_ = [("id", _L), ("start", _I), ("num_new", _I), ("samples", _I), ("rows_from", _I), ("num_rows", _I)]


class UpdateResult(Structure):
    _fields_ = [("id", _L), ("token", _I), ("reason", _I)]


class RequestInfo(Structure):
    _fields_ = [(n, _I) for n in ("num_prompt", "num_tokens", "num_computed", "status", "reason", "preemptions",
                                  "num_cached")]


_SIGNATURES = {
    "dh_pool_create": (_P, [_I]),
    "dh_pool_destroy": (None, [_P]),
    "dh_pool_num_free": (_I, [_P]),
    "dh_pool_allocate": (_I, [_P, _I, _P]),
    "dh_pool_free": (_I, [_P, _P, _I]),
    "dh_pool_free_list": (_I, [_P, _P, _I]),
    "dh_pool_is_held": (_I, [_P, _I]),
    "dh_pool_check": (_I, [_P]),
    "dh_cache_create": (_P, [_I, _P, _P, _P, _I, _I]),
    "dh_cache_lookup": (_L, [_P, _L, _P, _L]),
    "dh_cache_commit": (_I, [_P, _L, _P, _L]),
    "dh_cache_destroy": (None, [_P]),
    "dh_cache_has": (_I, [_P, _L]),
    "dh_cache_can_admit": (_I, [_P]),
    "dh_cache_admit": (_I, [_P, _L]),
    "dh_cache_take_fresh_slots": (_I, [_P, _P, _I]),
    "dh_cache_slot_of": (_I, [_P, _L]),
    "dh_cache_live_requests": (_I, [_P, _P, _I]),
    "dh_cache_pages_needed": (_I, [_P, _L, _L, _L, _P]),
    "dh_cache_allocate": (_I, [_P, _L, _L, _L]),
    "dh_cache_release_passed": (_I, [_P, _L, _L]),
    "dh_cache_free": (_I, [_P, _L]),
    "dh_cache_block_table": (_I, [_P, _L, _I, _P, _I]),
    "dh_cache_slot_mapping": (_I, [_P, _L, _I, _L, _L, _P]),
    "dh_cache_num_free": (_I, [_P, _I]),
    "dh_cache_free_list": (_I, [_P, _I, _P, _I]),
    "dh_cache_check": (_I, [_P]),
    "dh_batch_fill": (_I, [_P, POINTER(BatchBuffers), _I, _P, _P, _P, _P, _P, _P, _I, POINTER(BatchFacts)]),
    "dh_batch_pad": (_I, [POINTER(BatchBuffers), POINTER(BatchFacts), _I, _I, _I]),
    "dh_sched_create": (_P, [POINTER(SchedOptions), _P, _P, _I]),
    "dh_sched_destroy": (None, [_P]),
    "dh_sched_add": (_I, [_P, _L, _P, _I, _I, _I, _I, _P, _I, _I]),
    "dh_sched_abort": (_I, [_P, _L]),
    "dh_sched_forget": (_I, [_P, _L]),
    "dh_sched_has_unfinished": (_I, [_P]),
    "dh_sched_request_info": (_I, [_P, _L, POINTER(RequestInfo)]),
    "dh_sched_queue": (_I, [_P, _I, _P, _I]),
    "dh_sched_schedule": (_I, [_P, _P]),
    "dh_sched_can_look_ahead": (_I, [_P]),
    "dh_sched_schedule_ahead": (_I, [_P, _P]),
    "dh_sched_plan": (_I, [_P, _P, _P, _P, _P]),
    "dh_sched_fill": (_I, [_P, POINTER(BatchBuffers), _I, POINTER(BatchFacts)]),
    "dh_sched_update": (_I, [_P, _P, _I, _P, _I]),
}

_EXCEPTIONS = {1: KeyError, 2: RuntimeError, 3: ValueError, 4: AssertionError}
_fns: dict = {}
_last_error = None


def fn(name: str):
    f = _fns.get(name)
    if f is None:
        global _last_error
        lib = load_library("host")
        if _last_error is None:
            _last_error = lib.dh_last_error
            _last_error.restype, _last_error.argtypes = c_char_p, []
        restype, argtypes = _SIGNATURES[name]
        f = getattr(lib, name)
        f.restype, f.argtypes = restype, argtypes
        _fns[name] = f
    return f


def error(rc: int, context: str = "") -> Exception:
    """The Python exception for a negative status (the kind chooses the class)."""
    msg = _last_error().decode() if _last_error is not None else f"status {rc}"
    return _EXCEPTIONS.get(-rc, RuntimeError)(f"{context}{msg}")


def checked(name: str, *args, context: str = "") -> int:
    rc = fn(name)(*args)
    if rc < 0:
        raise error(rc, context)
    return rc


def created(name: str, *args):
    h = fn(name)(*args)
    if not h:
        msg = _last_error().decode() if _last_error is not None else ""
        raise ValueError(msg or f"{name} failed")
    return h
