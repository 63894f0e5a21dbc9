"""Continuous batching: admits requests, cuts prompts into portions under a token
budget, decodes, finishes and frees. Pure host code; it sees the cache only through
the cache manager. The rules are the reference's (crates/core/src/sched/mod.rs):

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

from collections import deque
from dataclasses import dataclass, field

from ..cache import CacheManager
from ..config import EngineOptions
from .request import FINISHED, LENGTH, PREEMPTED, RUNNING, STOP, WAITING, ABORT, Request


@dataclass
class ScheduledRequest:
    request: Request
    start: int       # tokens computed before this step
    num_new: int     # tokens this step feeds
    samples: bool    # the step reaches the end of the known tokens, so a token is sampled


@dataclass
class SchedulerOutput:
    scheduled: list = field(default_factory=list)      # [ScheduledRequest], running first then newly admitted
    preempted: list = field(default_factory=list)      # request ids preempted while scheduling
    force_finished: list = field(default_factory=list) # [(id, reason)] ended by the scheduler itself

    @property
    def total_tokens(self) -> int:
        return sum(s.num_new for s in self.scheduled)


class Scheduler:
    def __init__(self, options: EngineOptions, cache: CacheManager, eos_token_ids=()):
        self.opt, self.cache = options, cache
        self.eos = set(eos_token_ids)
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.requests: dict = {}

    # ---- intake --------------------------------------------------------------------------------
    def add_request(self, req: Request) -> None:
        if req.id in self.requests:
            raise KeyError(f"request id {req.id!r} is in use")
        if not req.prompt_ids:
            raise ValueError("a prompt needs at least one token")
        if req.num_prompt >= self.opt.max_model_len:
            raise ValueError(f"prompt of {req.num_prompt} tokens leaves no room for output within "
                             f"max_model_len {self.opt.max_model_len}")
        req.sampling.validate()
        req.status = WAITING
        self.requests[req.id] = req
        self.waiting.append(req)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def abort(self, req_id) -> None:
        req = self.requests.get(req_id)
        if req is None:
            return
        self._finish(req, ABORT)

    # ---- one step ------------------------------------------------------------------------------
    def schedule(self) -> SchedulerOutput:
        opt, out = self.opt, SchedulerOutput()
        budget = opt.max_num_batched_tokens
        quota = opt.prefill_tokens_per_step or (1 << 62)
        eligible = len(self.running) + len(self.waiting)
        threshold = opt.long_prefill_token_threshold if eligible > 1 else 0
        preempted_any = False

        i = 0
        while i < len(self.running):
            r = self.running[i]
            remaining = r.num_tokens - r.num_computed
            is_decode = remaining == 1 and r.num_computed > 0
            charged = not (opt.decode_exempt_from_budget and is_decode)
            if charged and budget == 0:
                break
            n = remaining
            if threshold and n > threshold:
                n = threshold
            if charged:
                n = min(n, budget)
            if not is_decode:
                n = min(n, quota)
            if n < remaining and not opt.enable_chunked_prefill:
                n = 0
            if n <= 0:
                i += 1
                continue
            got = False
            while True:
                if self.cache.allocate(r.id, r.num_computed, n):
                    got = True
                    break
                victim = self.running[-1]
                if victim is r:
                    if len(self.running) > 1:
                        break  # others hold the pages; try again next step, never preempt oneself
                    self._finish(r, LENGTH)  # alone and still no page: the pool cannot hold it
                    out.force_finished.append((r.id, LENGTH))
                    break
                self.running.pop()
                self._preempt(victim)
                out.preempted.append(victim.id)
                preempted_any = True
            if not got:
                break
            out.scheduled.append(ScheduledRequest(r, r.num_computed, n, r.num_computed + n == r.num_tokens))
            if charged:
                budget -= n
            if not is_decode:
                quota -= n
            i += 1

        if not preempted_any:
            while budget > 0 and self.waiting and len(self.running) < opt.max_num_seqs:
                r = self.waiting[0]
                remaining = r.num_tokens - r.num_computed
                n = remaining
                if threshold and n > threshold:
                    n = threshold
                n = min(n, budget, quota)
                if n < remaining and not opt.enable_chunked_prefill:
                    n = 0
                if n <= 0:
                    break
                if not self.cache.can_admit():
                    break
                self.cache.admit(r.id)
                if not self.cache.allocate(r.id, r.num_computed, n):
                    self.cache.free(r.id)  # no pages now: wait
                    break
                self.waiting.popleft()
                r.status = RUNNING
                self.running.append(r)
                out.scheduled.append(ScheduledRequest(r, r.num_computed, n, r.num_computed + n == r.num_tokens))
                budget -= n
                quota -= n

        for s in out.scheduled:  # advance at once, as the reference does after scheduling (:646-670)
            s.request.num_computed += s.num_new
        return out

    def update(self, out: SchedulerOutput, sampled: dict) -> list:
        """sampled: request id -> token for the scheduled requests that sample.
        Returns [(request, new token or None, finish reason or None)] for every scheduled request."""
        results = []
        for s in out.scheduled:
            r = s.request
            if r.status != RUNNING:
                continue  # preempted later in the same schedule() call
            self.cache.release_passed(r.id, r.num_computed)
            tok = None
            reason = None
            if s.samples:
                tok = int(sampled[r.id])
                r.output_ids.append(tok)
                reason = self._check_stop(r, tok)
                if reason:
                    self._finish(r, reason)
            results.append((r, tok, reason))
        return results

    # ---- internals -----------------------------------------------------------------------------
    def _check_stop(self, r: Request, tok: int) -> str | None:
        sp = r.sampling
        if r.num_output >= sp.min_tokens:
            if (not sp.ignore_eos and tok in self.eos) or tok in sp.stop_token_ids:
                return STOP
        if r.num_tokens >= self.opt.max_model_len or r.num_output >= sp.max_tokens:
            return LENGTH
        return None

    def _preempt(self, r: Request) -> None:
        self.cache.free(r.id)
        r.num_computed = 0
        r.status = PREEMPTED
        r.num_preemptions += 1
        self.waiting.appendleft(r)

    def _finish(self, r: Request, reason: str) -> None:
        if r.status == FINISHED:
            return
        if self.cache.has(r.id):
            self.cache.free(r.id)
        if r in self.running:
            self.running.remove(r)
        try:
            self.waiting.remove(r)
        except ValueError:
            pass
        r.status, r.finish_reason = FINISHED, reason
        self.requests.pop(r.id, None)
