"""Continuous batching: admits requests, cuts prompts into portions under a token
budget, decodes, finishes and frees. The decisions are made by the C++ class of
csrc/host/scheduler.hpp, which sees the cache only through the cache manager; this
front keeps the Python-side request objects and turns plans into Python values.
The rules are the reference's (crates/core/src/sched/mod.rs):

  * no separate prefill and decode phases: each step a request gets
    min(tokens it still has to compute, what the budget allows) tokens (:1-11,377);
  * running requests first, in admission order, then waiting ones first-come
    first-served while budget, request slots and pages last (:350-477);
  * a decode row (one token, with history) does not consume the budget when
    decode_exempt_from_budget is set (:351,361-365);
  * when pages run out for a running request, the last running request is preempted:
    its pages are freed, it forgets what it computed and goes to the front of the
    waiting queue, to recompute prompt and outputs later (:402-436,672-680). If the
    requester is itself the last one it is skipped this step while others run, and
    finished with "length" if it is alone (:414-432). A waiting request that cannot
    get pages waits (:571-573). A step that preempted admits nobody (:473);
  * finish: eos or stop id (after min_tokens, unless ignore_eos), max_tokens outputs,
    or max_model_len tokens (:816-828).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import numpy as np

from .. import native
from ..cache import CacheManager
from ..config import EngineOptions
from .request import REASON_NAMES, Request

_SCHEDULED = np.dtype([("id", "<i8"), ("start", "<i4"), ("num_new", "<i4"), ("samples", "<i4"), ("rows_from", "<i4"),
                       ("num_rows", "<i4")], align=True)
_RESULT = np.dtype([("id", "<i8"), ("token", "<i4"), ("reason", "<i4")], align=True)
assert _SCHEDULED.itemsize == ctypes.sizeof(native.Scheduled) and _RESULT.itemsize == ctypes.sizeof(native.UpdateResult)
_INT32_MAX = 2**31 - 1


@dataclass
class ScheduledRequest:
    request: Request
    start: int       # tokens computed before this step
    num_new: int     # tokens this step feeds
    samples: bool    # the step reaches the end of the known tokens, so a token is sampled


class SchedulerOutput:
    """One planned step. `rows` is the plan as the core wrote it (id, start, num_new, samples)."""

    def __init__(self, rows: np.ndarray, requests: list, preempted: list, force_finished: list):
        self.rows = rows
        self.requests = requests              # the Request of every row, running first then newly admitted
        self.preempted = preempted            # request ids preempted while scheduling
        self.force_finished = force_finished  # [(id, reason)] ended by the scheduler itself
        self._scheduled = None

    @property
    def scheduled(self) -> list:
        if self._scheduled is None:
            self._scheduled = [ScheduledRequest(r, int(x["start"]), int(x["num_new"]), bool(x["samples"]))
                               for r, x in zip(self.requests, self.rows)]
        return self._scheduled

    def __len__(self) -> int:
        return len(self.requests)

    @property
    def total_tokens(self) -> int:
        return int(self.rows["num_new"].sum())

    @property
    def single_rows_that_sample(self) -> bool:
        """Every request feeds one token and samples: the shape of a step that a captured graph replays."""
        return bool(len(self.rows)) and bool((self.rows["num_new"] == 1).all() and self.rows["samples"].all())

    def sampling_requests(self) -> list:
        return [r for r, s in zip(self.requests, self.rows["samples"].tolist()) if s]

    def prompt_rows(self) -> list:
        """[(request, position)]: the prompt positions at which this step returns logits beside the sampling rows
        (for requests that want the log-probabilities of their prompt), in the order of the logits rows that
        follow the sampling rows."""
        if not self.rows["num_rows"].any():
            return []
        return [(r, p) for r, lo, n in zip(self.requests, self.rows["rows_from"].tolist(), self.rows["num_rows"].tolist())
                for p in range(lo, lo + n)]


class Scheduler:
    def __init__(self, options: EngineOptions, cache: CacheManager, eos_token_ids=(), chunk_alignment: int | None = None):
        """chunk_alignment: where prompt portions may end (None: the options' own prefill_chunk_alignment; a runner
        passes that value raised to what its model's caches ask)."""
        self.opt, self.cache = options, cache
        self.eos = set(eos_token_ids)
        o = native.SchedOptions(options.max_num_batched_tokens, options.max_num_seqs, options.max_model_len,
                                options.prefill_tokens_per_step or 0, options.long_prefill_token_threshold or 0,
                                int(options.enable_chunked_prefill), int(options.decode_exempt_from_budget),
                                int(cache.prefix_caching if options.enable_prefix_caching is None
                                    else options.enable_prefix_caching), int(chunk_alignment or options.prefill_chunk_alignment or 1),
                                int(options.max_logits_rows or 0))
        eos = np.array(sorted(self.eos) or [0], dtype=np.int32)
        self._h = native.created("dh_sched_create", o, cache._h, eos.ctypes.data, len(self.eos))
        self.requests: dict = {}        # id -> Request, for every request that is not finished
        self._by_number: dict = {}      # the core's number -> Request
        self._info = native.RequestInfo()
        self._counts = (ctypes.c_int32 * 3)()
        cap = options.max_num_seqs
        self._results = np.zeros(cap, dtype=_RESULT)
        self._planned: list = []

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        try:
            if h:
                native.fn("dh_sched_destroy")(h)
        except Exception:  # the interpreter is shutting down: the process ends anyway
            pass

    # ---- intake --------------------------------------------------------------------------------
    def add_request(self, req: Request) -> None:
        if req.id in self.requests:
            raise KeyError(f"request id {req.id!r} is in use")
        if not req.prompt_ids:
            raise ValueError("a prompt needs at least one token")
        sp = req.sampling
        sp.validate()
        prompt = np.array(req.prompt_ids, dtype=np.int32)
        stop = np.array(list(sp.stop_token_ids) or [0], dtype=np.int32)
        number = self.cache.handle(req.id, create=True, pin=True)
        try:
            native.checked("dh_sched_add", self._h, number, prompt.ctypes.data, len(prompt),
                           min(sp.max_tokens, _INT32_MAX), sp.min_tokens, int(sp.ignore_eos), stop.ctypes.data,
                           len(sp.stop_token_ids), int(sp.prompt_logprobs is not None))
        except Exception:
            self.cache.forget(req.id)
            raise
        req._owner = self
        req._number = number
        self.requests[req.id] = req
        self._by_number[number] = req

    def has_unfinished(self) -> bool:
        return bool(native.fn("dh_sched_has_unfinished")(self._h))

    def abort(self, req_id) -> None:
        req = self.requests.get(req_id)
        if req is None:
            return
        native.checked("dh_sched_abort", self._h, req._number)
        self._release(req)

    def request_info(self, req: Request):
        native.checked("dh_sched_request_info", self._h, req._number, self._info)
        return self._info

    @property
    def waiting(self) -> list:
        return self._queue(0)

    @property
    def running(self) -> list:
        return self._queue(1)

    def _queue(self, running: int) -> list:
        cap = len(self.requests)
        out = np.zeros(max(cap, 1), dtype=np.int64)
        n = native.fn("dh_sched_queue")(self._h, running, out.ctypes.data, cap)
        return [self._by_number[h] for h in out[:n].tolist()]

    # ---- one step ------------------------------------------------------------------------------
    def can_look_ahead(self) -> bool:
        """The step planned last has not been updated yet (it is running), and the one after it can be planned now:
        it feeds one token of every request and samples each, nobody waits to be admitted, and pages are at hand, so
        the next step is every request decoding once more (crates/core/src/sched/mod.rs:8-9,646-670)."""
        return bool(native.checked("dh_sched_can_look_ahead", self._h))

    def schedule(self, ahead: bool = False) -> SchedulerOutput:
        """ahead: plan the step after the one that still runs (can_look_ahead()); each request's input token is then
        the one the running step samples, a placeholder here. update() then applies to the running step first."""
        native.checked("dh_sched_schedule_ahead" if ahead else "dh_sched_schedule", self._h, self._counts)
        n, n_pre, n_fin = self._counts
        rows = np.zeros(n, dtype=_SCHEDULED)
        pre = np.zeros(max(n_pre, 1), dtype=np.int64)
        fin = np.zeros(max(n_fin, 1), dtype=np.int64)
        why = np.zeros(max(n_fin, 1), dtype=np.int32)
        native.fn("dh_sched_plan")(self._h, rows.ctypes.data, pre.ctypes.data, fin.ctypes.data, why.ctypes.data)
        by = self._by_number
        requests = [by[h] for h in rows["id"].tolist()]
        preempted = [by[h].id for h in pre[:n_pre].tolist()]
        forced = []
        for h, reason in zip(fin[:n_fin].tolist(), why[:n_fin].tolist()):
            r = by[h]
            forced.append((r.id, REASON_NAMES[reason]))
            self._release(r)
        self._planned = requests
        return SchedulerOutput(rows, requests, preempted, forced)

    def planned_ids(self) -> list:
        return [r.id for r in self._planned]

    def update(self, out: SchedulerOutput, sampled) -> list:
        """sampled: request id -> token for the scheduled requests that sample, or the tokens alone
        in the order of those requests. Returns [(request, new token or None, finish reason or None)]
        for every scheduled request that is still running."""
        if isinstance(sampled, dict):
            sampled = [sampled[r.id] for r in out.sampling_requests()]
        toks = np.array(list(sampled) or [0], dtype=np.int32)
        if len(self._results) < len(out):
            self._results = np.zeros(len(out), dtype=_RESULT)
        n = native.checked("dh_sched_update", self._h, toks.ctypes.data, len(sampled), self._results.ctypes.data,
                           len(self._results))
        res = self._results[:n]
        results = []
        by = self._by_number
        for h, tok, reason in zip(res["id"].tolist(), res["token"].tolist(), res["reason"].tolist()):
            r = by[h]
            if tok >= 0:
                r.output_ids.append(tok)
            else:
                tok = None
            if reason:
                self._release(r)
            results.append((r, tok, REASON_NAMES[reason]))
        return results

    # ---- internals -----------------------------------------------------------------------------
    def _release(self, req: Request) -> None:
        """A finished request: keep its last state on the Python object, drop it from the core."""
        req._detach(self.request_info(req))
        native.checked("dh_sched_forget", self._h, req._number)
        self.requests.pop(req.id, None)
        self._by_number.pop(req._number, None)
        self.cache.forget(req.id)
