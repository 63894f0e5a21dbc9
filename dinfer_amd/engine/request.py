"""A request's life: its tokens, how many of them are computed, and why it ended
(crates/core/src/request.rs:8-159).

The prompt, the outputs, the sampling parameters and the seed live here. While a
scheduler owns the request, the counters that scheduling changes (tokens computed,
status, preemptions) are read from the C++ core, which is the only writer; when
the request finishes its last state is copied back here.
"""
from __future__ import annotations

from ..sampling.params import SamplingParams

WAITING, RUNNING, PREEMPTED, FINISHED = "waiting", "running", "preempted", "finished"
STOP, LENGTH, ABORT = "stop", "length", "abort"
STATUS_NAMES = (WAITING, RUNNING, PREEMPTED, FINISHED)
REASON_NAMES = (None, STOP, LENGTH, ABORT)


class Request:
    def __init__(self, id, prompt_ids: list, sampling: SamplingParams, seed: int = 0):
        self.id = id
        self.prompt_ids = prompt_ids
        self.sampling = sampling
        self.seed = seed
        self.output_ids: list = []
        self._owner = None            # the scheduler that holds the live counters
        self._num_computed = 0
        self._status = WAITING
        self._finish_reason: str | None = None
        self._num_preemptions = 0
        self._num_cached = 0

    def __repr__(self) -> str:
        return (f"Request(id={self.id!r}, prompt={self.num_prompt}, outputs={self.num_output}, "
                f"computed={self.num_computed}, status={self.status})")

    # ---- counters the scheduler changes
    def _live(self):
        return self._owner.request_info(self) if self._owner is not None else None

    @property
    def num_computed(self) -> int:
        info = self._live()
        return info.num_computed if info else self._num_computed

    @property
    def status(self) -> str:
        info = self._live()
        return STATUS_NAMES[info.status] if info else self._status

    @property
    def finish_reason(self) -> str | None:
        info = self._live()
        return REASON_NAMES[info.reason] if info else self._finish_reason

    @property
    def num_preemptions(self) -> int:
        info = self._live()
        return info.preemptions if info else self._num_preemptions

    @property
    def num_cached_tokens(self) -> int:
        """Tokens found in the prefix cache when the request was last admitted (not computed again)."""
        info = self._live()
        return info.num_cached if info else self._num_cached

    def _detach(self, info) -> None:
        """Keeps the last state when the scheduler lets the request go."""
        self._num_computed, self._status = info.num_computed, STATUS_NAMES[info.status]
        self._finish_reason, self._num_preemptions = REASON_NAMES[info.reason], info.preemptions
        self._num_cached = info.num_cached
        self._owner = None

    # ---- tokens
    @property
    def num_prompt(self) -> int:
        return len(self.prompt_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.output_ids)

    @property
    def num_output(self) -> int:
        return len(self.output_ids)

    def tokens(self, start: int, n: int) -> list:
        p = self.num_prompt
        if start + n <= p:
            return self.prompt_ids[start:start + n]
        if start >= p:
            return self.output_ids[start - p:start - p + n]
        return self.prompt_ids[start:] + self.output_ids[:start + n - p]
