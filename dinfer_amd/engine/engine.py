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
        self.scheduler = Scheduler(self.options, self.runner.cache, spec.eos_token_ids)
        self.sampler = Sampler(self.runner.device, self.runner.max_rows, spec.vocab_size)
        self._ids = itertools.count()
        self._seeds = random.Random()
        self.phases: dict | None = None     # see measure_phases

    # ---- requests ------------------------------------------------------------------------------
    def add_request(self, prompt_ids: list, sampling: SamplingParams | None = None, request_id=None):
        sampling = sampling or SamplingParams()
        bad = [t for t in prompt_ids if not (isinstance(t, int) and 0 <= t < self.vocab_size)]
        if bad:
            raise ValueError(f"token {bad[0]!r} is outside the vocabulary of {self.vocab_size}")
        rid = next(self._ids) if request_id is None else request_id
        seed = sampling.seed if sampling.seed is not None else self._seeds.getrandbits(64)
        self.scheduler.add_request(Request(rid, list(prompt_ids), sampling, seed=seed))
        return rid

    def abort(self, request_id) -> None:
        self.scheduler.abort(request_id)
        self.sampler.forget(request_id)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    # ---- one step ------------------------------------------------------------------------------
    def step(self) -> list[StepOutput]:
        if self.phases is not None:
            return self._step_timed()
        so = self.scheduler.schedule()
        outs = [StepOutput(rid, None, True, reason) for rid, reason in so.force_finished]
        if not len(so):
            return outs
        logits = self.runner.step_planned(self.scheduler, so)
        rows = [(r.sampling, len(r.output_ids), r.prompt_ids, r.output_ids, r.seed, r.id) for r in so.sampling_requests()]
        tokens = self.sampler.sample(logits, rows)
        for r, tok, reason in self.scheduler.update(so, tokens):
            outs.append(StepOutput(r.id, tok, reason is not None, reason))
        for o in outs:
            if o.finished:
                self.sampler.forget(o.request_id)
        return outs

    def measure_phases(self, on: bool = True) -> None:
        """From now on every step adds its host times to `phases` (seconds; the reference accounts a step the same way,
        models/qwen3/src/executor.rs:150-157,734-748): schedule (the plan), fill (batch written and sent), launch
        (graph replay or kernel launches issued), sample (sampling kernels issued), wait (the host waits for the tokens:
        what the GPU still has to do once everything is issued), update (requests advanced, pages released), and
        gpu (the model's kernels on the device, between two events); steps counts them."""
        self.phases = {k: 0.0 for k in ("schedule", "fill", "launch", "sample", "wait", "update", "gpu")} if on else None
        if on:
            self.phases["steps"] = 0
        self.runner.phases = self.sampler.phases = self.phases

    def _step_timed(self) -> list[StepOutput]:
        import time
        ph, t = self.phases, time.perf_counter
        t0 = t()
        so = self.scheduler.schedule()
        ph["schedule"] += t() - t0
        outs = [StepOutput(rid, None, True, reason) for rid, reason in so.force_finished]
        if not len(so):
            return outs
        logits = self.runner.step_planned(self.scheduler, so)          # adds to fill and launch itself
        rows = [(r.sampling, len(r.output_ids), r.prompt_ids, r.output_ids, r.seed, r.id) for r in so.sampling_requests()]
        tokens = self.sampler.sample(logits, rows)                     # adds to sample and wait itself
        t0 = t()
        for r, tok, reason in self.scheduler.update(so, tokens):
            outs.append(StepOutput(r.id, tok, reason is not None, reason))
        for o in outs:
            if o.finished:
                self.sampler.forget(o.request_id)
        ph["update"] += t() - t0
        ph["steps"] += 1
        ev = self.runner.take_gpu_events()
        if ev is not None:
            ev[1].synchronize()        # a step in which nobody samples has not waited for the device yet
            ph["gpu"] += ev[0].elapsed_time(ev[1]) * 1e-3
        return outs

    def generate(self, prompts: list, sampling: SamplingParams | list | None = None) -> list[list[int]]:
        """Runs the prompts (lists of token ids) to the end; returns the generated ids of each."""
        params = sampling if isinstance(sampling, list) else [sampling or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        got = {i: [] for i in ids}
        idle = 0
        while self.has_unfinished():
            outs = self.step()
            idle = 0 if outs else idle + 1
            if idle > 2:
                raise RuntimeError("the scheduler made no progress: a request fits neither the budget nor the pool")
            for o in outs:
                if o.token is not None and o.request_id in got:
                    got[o.request_id].append(o.token)
        return [got[i] for i in ids]
