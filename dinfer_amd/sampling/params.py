"""Sampling options of a request: names, defaults and ranges of the reference's
SamplingParams (crates/core/src/sample.rs:81-139, validate :157-205), without the
text-level and server-level fields (stop strings, grammar).
"""
from __future__ import annotations

from dataclasses import dataclass, field

GREEDY_EPS = 1e-5  # temperature at or below this is greedy (sample.rs:143-145)
MAX_LOGPROBS = 20      # sample.rs:184-188
MAX_LOGIT_BIAS = 300   # entries, each in [-100, 100] (sample.rs:198-203)


@dataclass
class TokenLogprobs:
    """What a request with `logprobs` gets beside every output token (crates/core/src/sampler.rs:156-166)."""
    token_id: int
    logprob: float       # log_softmax(the model's logits)[token_id]: before logit_bias, penalties and temperature
    rank: int            # how many tokens have a larger logit (0: it is the most probable one)
    top: list            # the k most probable (token id, logprob), falling


@dataclass
class SamplingParams:
    max_tokens: int = 256
    min_tokens: int = 0            # eos / stop ids are ignored until this many outputs
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = -1
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    seed: int | None = None        # None: drawn at admission
    stop_token_ids: list = field(default_factory=list)
    ignore_eos: bool = False
    logprobs: int | None = None    # k: every output token comes with its log-probability, its rank and the k most
                                   # probable tokens (0: only its own), from the logits the model produced
    logit_bias: dict = field(default_factory=dict)   # token id -> what is added to its logit before anything else
                                                     # (pairs (token, bias) are taken too)
    prompt_logprobs: int | None = None   # k: the same for every token of the prompt but the first, given the
                                         # tokens before it (the engine needs max_logits_rows > max_num_seqs)

    def __post_init__(self):
        pairs = list(self.logit_bias.items()) if isinstance(self.logit_bias, dict) else list(self.logit_bias)
        as_dict = {int(t): float(b) for t, b in pairs}       # (keys may come as strings of digits)
        if len(as_dict) != len(pairs):
            raise ValueError("logit_bias names a token twice")
        self.logit_bias = as_dict

    @property
    def is_greedy(self) -> bool:
        return self.temperature <= GREEDY_EPS

    @property
    def picks_largest_logit(self) -> bool:
        """The token is the largest of the logits the model produced: nothing changes them on the way."""
        return self.is_greedy and not self.has_penalties and not self.logit_bias

    @property
    def has_penalties(self) -> bool:
        return self.repetition_penalty != 1.0 or self.frequency_penalty != 0.0 or self.presence_penalty != 0.0

    def validate(self) -> None:
        if self.temperature < 0.0:
            raise ValueError(f"temperature must be non-negative, got {self.temperature}")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if self.top_k < -1 or self.top_k == 0:
            raise ValueError(f"top_k must be -1 (disable) or at least 1, got {self.top_k}")
        if not (0.0 <= self.min_p <= 1.0):
            raise ValueError(f"min_p must be in [0, 1], got {self.min_p}")
        if not (0.0 < self.repetition_penalty <= 2.0):
            raise ValueError(f"repetition_penalty must be in (0, 2], got {self.repetition_penalty}")
        if not (-2.0 <= self.frequency_penalty <= 2.0):
            raise ValueError(f"frequency_penalty must be in [-2, 2], got {self.frequency_penalty}")
        if not (-2.0 <= self.presence_penalty <= 2.0):
            raise ValueError(f"presence_penalty must be in [-2, 2], got {self.presence_penalty}")
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.min_tokens > self.max_tokens:
            raise ValueError(f"min_tokens {self.min_tokens} > max_tokens {self.max_tokens}")
        if self.logprobs is not None and not (0 <= self.logprobs <= MAX_LOGPROBS):
            raise ValueError(f"logprobs must be in [0, {MAX_LOGPROBS}], got {self.logprobs}")
        if self.prompt_logprobs is not None and not (0 <= self.prompt_logprobs <= MAX_LOGPROBS):
            raise ValueError(f"prompt_logprobs must be in [0, {MAX_LOGPROBS}], got {self.prompt_logprobs}")
        if len(self.logit_bias) > MAX_LOGIT_BIAS:
            raise ValueError(f"logit_bias has {len(self.logit_bias)} entries, at most {MAX_LOGIT_BIAS}")
        for t, b in self.logit_bias.items():
            if not (isinstance(t, int) and t >= 0):
                raise ValueError(f"logit_bias names {t!r}, which is no token id")
            if not (-100.0 <= b <= 100.0):
                raise ValueError(f"logit_bias[{t}] = {b} is outside [-100, 100]")
        if self.seed is not None and not (0 <= self.seed < 1 << 64):
            raise ValueError(f"seed must fit 64 unsigned bits, got {self.seed}")
