"""The Python entry point: an engine that owns runner, scheduler and sampler.

    engine = Engine("model_dir", dtype="bfloat16", max_num_seqs=16)
    outputs = engine.generate([[1, 2, 3], [4, 5]], SamplingParams(max_tokens=8, temperature=0))

``add_request`` / ``step`` drive it one step at a time: schedule -> build the batch ->
one step of the model -> sample -> update (crates/core/src/engine.rs:538-729 without
the server thread; the run-until-empty loop is the one of
models/qwen3/tests/real_parity.rs:246-255).
"""
from __future__ import annotations

import itertools
import random
import time
from dataclasses import dataclass

from ..config import EngineOptions
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .request import Request
from .runner import ModelRunner
from .scheduler import Scheduler


@dataclass
class StepOutput:
    request_id: object
    token: int | None          # None: a portion of a prompt was computed, nothing sampled
    finished: bool
    finish_reason: str | None
    logprobs: object = None    # TokenLogprobs of the token, for a request that asked for them
    prompt_logprobs: list | None = None   # [(position, TokenLogprobs)] of the prompt tokens this step judged


@dataclass
class Generation:
    """What generate(..., details=True) returns for a prompt."""
    token_ids: list
    finish_reason: str | None
    logprobs: list | None          # one TokenLogprobs per generated token (SamplingParams.logprobs)
    prompt_logprobs: list | None   # one per prompt token, None for the first (SamplingParams.prompt_logprobs)


@dataclass
class _InFlight:
    """A step that has been launched and whose tokens have not been read yet."""
    plan: object                    # the scheduler's plan of the step
    sampled: object                 # Sampler.launch's handle: the tokens on their way
    events: tuple | None            # device events around the model's kernels (while phases are measured)
    asking: list | None             # the sampled rows' requests, if one of them wants log-probabilities
    prompt_rows: list | None        # [(request, position)] of the prompt positions judged in this step
    prompt_found: object = None     # Sampler.about_rows' handle for them


_ENDED = {"stop": "request_success_stop", "length": "request_success_length", "abort": "request_abort"}


class _Ready:
    """Tokens that are on the host already, in the shape of what Sampler.launch returns."""

    def __init__(self, tokens):
        self._tokens = tokens

    def tokens(self):
        return self._tokens

    def logprobs(self):
        return [None] * len(self._tokens)


class Engine:
    def __init__(self, model: str | None = None, *, config=None, seed: int = 0, runner: ModelRunner | None = None,
                 options: EngineOptions | None = None, **option_fields):
        """model: a folder with config.json and safetensors. Or config=<typed configuration> with
        seed: random weights drawn on the device. Engine options by keyword (see EngineOptions)."""
        opt = options or EngineOptions(**option_fields)
        if runner is not None:
            self.runner = runner
        elif model is not None:
            self.runner = ModelRunner.from_dir(model, opt)
        elif config is not None:
            self.runner = ModelRunner.from_config(config, opt, seed)
        else:
            raise ValueError("give a model folder, a configuration, or a runner")
        self.options = self.runner.options
        spec = self.runner.model.spec
        self.vocab_size = spec.vocab_size
        self.scheduler = Scheduler(self.options, self.runner.cache, spec.eos_token_ids,
                                   chunk_alignment=getattr(self.runner, "chunk_alignment", None))
        # the sampled tokens land where the next step can take them from as its input, if it is launched before
        # the host has read them
        last = getattr(getattr(self.runner, "batch", None), "last_tokens", None)
        # a step samples one row per request at most; the rows beyond that are prompt positions to be judged
        rows = self.runner.max_rows
        self.sampler = Sampler(self.runner.device, min(rows, self.options.max_num_seqs), spec.vocab_size, out=last,
                               max_judged=rows)
        self._running: _InFlight | None = None      # the step whose tokens are read next
        self._ids = itertools.count()
        self._seeds = random.Random()
        # counters under the names of the reference's engine metrics (crates/core/src/metrics.rs:63-89)
        self.counters = {k: 0 for k in ("engine_steps_total", "prompt_tokens_total", "generation_tokens_total",
                                        "num_preemptions_total", "prefix_cache_hit_tokens_total", "request_success_stop",
                                        "request_success_length", "request_abort")}
        self._in_prompt: set = set()        # requests with prompt tokens still to compute (what the counters look at)
        self.steps_launched_ahead = 0       # steps issued before the tokens of the step before them were read
        self.phases: dict | None = None     # see measure_phases

    # ---- requests ------------------------------------------------------------------------------
    def add_request(self, prompt_ids: list, sampling: SamplingParams | None = None, request_id=None):
        sampling = sampling or SamplingParams()
        bad = [t for t in prompt_ids if not (isinstance(t, int) and 0 <= t < self.vocab_size)]
        bad += [t for t in sampling.logit_bias if not 0 <= t < self.vocab_size]
        if bad:
            raise ValueError(f"token {bad[0]!r} is outside the vocabulary of {self.vocab_size}")
        rid = next(self._ids) if request_id is None else request_id
        seed = sampling.seed if sampling.seed is not None else self._seeds.getrandbits(64)
        self.scheduler.add_request(Request(rid, list(prompt_ids), sampling, seed=seed))
        self._in_prompt.add(rid)
        return rid

    def abort(self, request_id) -> None:
        if request_id in self.scheduler.requests:
            self.counters["request_abort"] += 1
        self.scheduler.abort(request_id)
        self.sampler.forget(request_id)
        self._in_prompt.discard(request_id)

    def stats(self) -> dict:
        """The counters since the engine was made, and what is true now: requests running and waiting, and the
        share of the cache's pages in use (of the fullest group)."""
        cache = self.runner.cache
        used = [1.0 - cache.num_free(g) / max(spec.num_blocks, 1) for g, spec in enumerate(cache.groups)]
        return dict(self.counters, num_requests_running=len(self.scheduler.running),
                    num_requests_waiting=len(self.scheduler.waiting), kv_cache_usage=max(used, default=0.0))

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished() or self._running is not None

    # ---- one step ------------------------------------------------------------------------------
    def step(self) -> list[StepOutput]:
        """Plans, runs and samples one step and returns what it brought. With async_scheduling, where that step is
        one of single decode rows, the step after it is planned and launched before this one's tokens are read, and
        stays in flight when this call returns (crates/core/src/engine.rs:538-729)."""
        ph = self.phases
        outs: list = []
        if self._running is None:
            outs = self._launch(ahead=False)
            if self._running is None:
                return outs               # nothing was scheduled
        nxt = None
        if self._may_look_ahead():
            self._running, held = None, self._running
            try:
                outs += self._launch(ahead=True)        # (a plan ahead ends nobody: nothing is added)
                self.steps_launched_ahead += 1
            finally:                                    # whatever happened, the running step is still the running step
                self._running, nxt = held, self._running
        run = self._running
        events = run.events
        tokens = run.sampled.tokens()
        t0 = time.perf_counter() if ph is not None else 0.0
        about, about_prompt = {}, {}
        if run.asking is not None:
            about = {r.id: lp for r, lp in zip(run.asking, run.sampled.logprobs()) if lp is not None}
        if run.prompt_rows:
            for (r, pos), lp in zip(run.prompt_rows, run.prompt_found.logprobs()):
                about_prompt.setdefault(r.id, []).append((pos + 1, lp))       # the token judged is the next one
        count = self.counters
        for r, tok, reason in self.scheduler.update(run.plan, tokens):
            outs.append(StepOutput(r.id, tok, reason is not None, reason, about.get(r.id) if tok is not None else None,
                                   about_prompt.get(r.id)))
            count["generation_tokens_total"] += tok is not None
            if reason is not None:
                count[_ENDED[reason]] += 1
        for o in outs:
            if o.finished:
                self.sampler.forget(o.request_id)
        self._running = nxt
        if ph is not None:
            ph["update"] += time.perf_counter() - t0
            ph["steps"] += 1
            if events is not None:
                events[1].synchronize()        # a step in which nobody samples has not waited for the device yet
                ph["gpu"] += events[0].elapsed_time(events[1]) * 1e-3
        return outs

    def _may_look_ahead(self) -> bool:
        """The step after the running one can be launched before the running one's tokens are read: the scheduler
        can plan it (everyone decodes once more), and no row needs the token on the host to sample the next (a
        penalty counts the tokens seen so far)."""
        if not self.options.async_scheduling or not self.scheduler.can_look_ahead():
            return False
        return not any(r.sampling.has_penalties for r in self._running.plan.requests)

    def _launch(self, ahead: bool) -> list[StepOutput]:
        """Plans a step and issues it and its sampling; what is in flight afterwards is in _running (None: nothing
        was scheduled). Returns the outputs of requests the scheduler itself ended while planning."""
        ph = self.phases
        t0 = time.perf_counter() if ph is not None else 0.0
        so = self.scheduler.schedule(ahead=ahead)
        if ph is not None:
            ph["schedule"] += time.perf_counter() - t0
        outs = [StepOutput(rid, None, True, reason) for rid, reason in so.force_finished]
        count = self.counters
        count["num_preemptions_total"] += len(so.preempted)
        self._in_prompt.update(so.preempted)        # (they compute their prompts again)
        for rid, reason in so.force_finished:
            count[_ENDED[reason]] += 1
            self._in_prompt.discard(rid)
        if not len(so):
            self._running = None
            return outs
        count["engine_steps_total"] += 1
        if self._in_prompt:
            for x in so.scheduled:
                r = x.request
                if r.id not in self._in_prompt:
                    continue
                count["prompt_tokens_total"] += max(0, min(x.start + x.num_new, r.num_prompt) - x.start)
                if x.start and x.start == r.num_cached_tokens:      # admitted in this step with that many found
                    count["prefix_cache_hit_tokens_total"] += x.start
                if x.start + x.num_new >= r.num_prompt:
                    self._in_prompt.discard(r.id)
        sampling = so.sampling_requests()
        greedy = all(r.sampling.picks_largest_logit for r in sampling)
        logits = self.runner.step_planned(self.scheduler, so, greedy=greedy)      # adds to fill and launch itself
        # a request whose last token is still on its way has produced one more than its list says
        rows = [(r.sampling, len(r.output_ids) + (1 if ahead else 0), r.prompt_ids, r.output_ids, r.seed, r.id)
                for r in sampling]
        launch = getattr(self.sampler, "launch", None)                 # (a stand-in may only know how to sample())
        ours = logits[:len(rows)]       # (rows of prompt positions may follow)
        if launch:      # adds to sample (and, later, to wait); a replayed graph may have found the best tokens already
            sampled = launch(ours, rows, done=getattr(self.runner, "argmax_done", False))
        else:
            sampled = _Ready(self.sampler.sample(ours, rows))
        asking = sampling if any(r.sampling.logprobs is not None for r in sampling) else None
        prompt, found = so.prompt_rows(), None
        if prompt:      # their logits follow the sampling rows
            found = self.sampler.about_rows(logits[len(rows):len(rows) + len(prompt)],
                                            [r.prompt_ids[p + 1] for r, p in prompt],
                                            [r.sampling.prompt_logprobs for r, _ in prompt])
        self._running = _InFlight(so, sampled, self.runner.take_gpu_events() if ph is not None else None, asking,
                                  prompt, found)
        return outs

    def measure_phases(self, on: bool = True) -> None:
        """From now on every step adds its host times to `phases` (seconds; the reference accounts a step the same way,
        models/qwen3/src/executor.rs:150-157,734-748): schedule (the plan), fill (batch written and sent), launch
        (graph replay or kernel launches issued), sample (sampling kernels issued), wait (the host stands still until
        the tokens of the oldest step in flight are there), update (requests advanced, pages released), and gpu (the
        model's kernels on the device, between two events); steps counts them."""
        self.phases = {k: 0.0 for k in ("schedule", "fill", "launch", "sample", "wait", "update", "gpu")} if on else None
        if on:
            self.phases["steps"] = 0
        self.runner.phases = self.sampler.phases = self.phases

    def generate(self, prompts: list, sampling: SamplingParams | list | None = None, *, details: bool = False):
        """Runs the prompts (lists of token ids) to the end; returns the generated ids of each, or with `details`
        a Generation for each (ids, finish reason, and the log-probabilities its SamplingParams asked for)."""
        params = sampling if isinstance(sampling, list) else [sampling or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        got = {i: [] for i in ids}
        about = {i: [] for i in ids}
        about_prompt = {i: [None] for i in ids}
        why = {i: None for i in ids}
        idle = 0
        while self.has_unfinished():
            outs = self.step()
            idle = 0 if outs else idle + 1
            if idle > 2:
                raise RuntimeError("the scheduler made no progress: a request fits neither the budget nor the pool")
            for o in outs:
                if o.request_id not in got:
                    continue
                if o.token is not None:
                    got[o.request_id].append(o.token)
                    about[o.request_id].append(o.logprobs)
                for pos, lp in o.prompt_logprobs or ():
                    assert pos == len(about_prompt[o.request_id]), "prompt positions come in order, each once"
                    about_prompt[o.request_id].append(lp)
                if o.finished:
                    why[o.request_id] = o.finish_reason
        if details:
            return [Generation(got[i], why[i], about[i] if p.logprobs is not None else None,
                               about_prompt[i] if p.prompt_logprobs is not None else None)
                    for i, p in zip(ids, params)]
        return [got[i] for i in ids]
