"""A request's life: its tokens, how many of them are computed, and why it ended
(crates/core/src/request.rs:8-159)."""
from __future__ import annotations

from dataclasses import dataclass, field

from ..sampling.params import SamplingParams

WAITING, RUNNING, PREEMPTED, FINISHED = "waiting", "running", "preempted", "finished"
STOP, LENGTH, ABORT = "stop", "length", "abort"


@dataclass
class Request:
    id: object
    prompt_ids: list
    sampling: SamplingParams
    seed: int = 0
    output_ids: list = field(default_factory=list)
    num_computed: int = 0
    status: str = WAITING
    finish_reason: str | None = None
    num_preemptions: int = 0

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
