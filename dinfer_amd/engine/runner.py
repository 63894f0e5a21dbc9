"""The model runner: owns the model, the cache pages and the step function.

``step(entries)`` is the one step function of the engine: it runs exactly the
tokens it is given, as one batch, against the cache that earlier steps left, and
returns the logits at the wanted places. Generation, the scheduler's engine loop
and trace replay all go through it; none of them has a forward pass, a cache or
a loader of its own (models/qwen3/src/executor.rs:977-1031, model.rs:684-832).
"""
from __future__ import annotations

from pathlib import Path

import torch

from ..cache import CacheManager, GroupSpec
from ..config import EngineOptions, load_config
from ..kernels import blaslt, gemm, ops
from ..parts import BuildContext, CacheView, DecoderModel
from ..weights import WeightLoader
from .batch import Entry, StepBatch

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _require_gpu(device_index: int) -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("dinfer_amd needs a GPU: no HIP device is visible and there is no CPU path")
    if device_index >= torch.cuda.device_count():
        raise RuntimeError(f"device {device_index} does not exist ({torch.cuda.device_count()} visible)")
    dev = torch.device("cuda", device_index)
    torch.cuda.set_device(dev)
    return dev


_first_graph_done: set = set()


def _first_graph(device) -> None:
    """Instantiates one tiny HIP graph per device before any other, captured by hand (torch's capture context
    empties the allocator's cache first, which is what must not have happened yet).

    Measured on MI355X with ROCm 7: every decode graph of the process replays faster afterwards, the more the
    more kernels it holds (8B sizes: 8.6 -> 8.2 ms a step at batch 64, 330 kernels of 5 to 95 us; nothing at batch 8),
    with the same kernels at the same durations under the profiler, so the difference lies between them. When the
    first graph the runtime instantiates is a decode graph itself, or any graph after the allocator's cache has
    been emptied, all later ones stay slow. The cause inside the runtime is not known; the order is cheap to keep."""
    if device in _first_graph_done:
        return
    _first_graph_done.add(device)
    with torch.cuda.device(device):
        cell = torch.zeros(64, dtype=torch.float32, device=device)
        side = torch.cuda.Stream(device=device)
        graph = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            graph.capture_begin()
            try:
                ops.fill_zero(cell)
            finally:
                graph.capture_end()
        torch.cuda.current_stream().wait_stream(side)
        graph.replay()
        torch.cuda.synchronize(device)


class ModelRunner:
    def __init__(self, model: DecoderModel, options: EngineOptions, device: torch.device):
        options.check()
        self.model, self.options, self.device = model, options, device
        self.dtype = _DTYPES[options.dtype]
        spec = model.spec
        if options.max_model_len > spec.max_positions:
            raise ValueError(f"max_model_len {options.max_model_len} exceeds the model's "
                             f"{spec.max_positions} positions")
        self.page_size = options.block_size
        self.max_rows = options.max_logits_rows or options.max_num_seqs
        # decode rows may ride on top of the prompt budget (service.rs:206-210)
        self.max_tokens = options.max_num_batched_tokens + (options.max_num_seqs if options.decode_exempt_from_budget else 0)
        self.ctx = BuildContext(device, self.dtype, self.max_tokens, self.max_rows, self.page_size,
                                options.max_num_seqs, max_seq_len=options.max_model_len)
        blaslt.configure(tuning=options.gemm_tuning, plan_file=options.gemm_plan_file)
        if self.dtype == torch.bfloat16:
            blaslt.require()
        model.bind(self.ctx)
        self._build_caches()
        self.batch = StepBatch(device, self.max_tokens, options.max_num_seqs, self.max_rows,
                               [self.max_blocks_per_seq] * len(self.group_specs))
        # batch-size buckets of the decode graphs: powers of two; between 16 and 64 every multiple of 8 (the few-row
        # products load the activations row by row: at the 8B sizes a step of 24 rows takes 5.5 ms in a graph of 24
        # and 5.7 ms in one of 32); beyond, the step between two powers as well; and the largest batch
        top = min(options.max_num_seqs, self.max_rows, self.max_tokens)
        sizes = {1 << i for i in range(top.bit_length() + 1)} | {24, 40, 48, 56} | {3 << i for i in range(5, top.bit_length())}
        self._buckets = sorted({min(x, top) for x in sizes})
        self._graphs: dict[tuple, torch.cuda.CUDAGraph] = {}   # (bucket, finds the best tokens itself) -> graph
        self._argmax_scratch: torch.Tensor | None = None       # made in the eager step before the first such capture
        self.phases: dict | None = None     # Engine.measure_phases
        self._events = None
        self._graph_pool = None
        self._capture_stream = None
        # a step is replayed from a graph only where every part reads what changes between steps from device memory
        self._graphs_allowed = bool(options.hip_graph) and model.capturable()
        # steps with prompt portions: padded up to a few counts, and replayed from a graph of their own once the same
        # counts have come up PORTION_GRAPH_AFTER times (a capture costs about two eager steps)
        self._portion_graphs_allowed = self._graphs_allowed and model.capturable_portions()
        self._portion_graphs: dict[tuple, torch.cuda.CUDAGraph] = {}
        self._portion_seen: dict[tuple, int] = {}
        self.portion_replays = 0            # steps with prompt portions served by a replay
        if self._graphs_allowed and self.device.type == "cuda":
            _first_graph(self.device)
        self.warm_up()

    # ---- construction --------------------------------------------------------------------------
    @classmethod
    def from_dir(cls, model_dir: str | Path, options: EngineOptions) -> "ModelRunner":
        device = _require_gpu(options.device)
        arch, cfg = load_config(model_dir)
        model = DecoderModel(arch.build_spec(cfg))
        loader = WeightLoader(model_dir, device, _DTYPES[options.dtype])
        try:
            model.load(loader)
        finally:
            loader.close()
        r = cls(model, options, device)
        r.config = cfg
        return r

    @classmethod
    def from_config(cls, cfg, options: EngineOptions, seed: int = 0) -> "ModelRunner":
        """Random weights drawn on the device (measurements; no file is written)."""
        from ..config import get_architecture
        device = _require_gpu(options.device)
        model = DecoderModel(get_architecture(cfg.ARCHITECTURE).build_spec(cfg))
        model.load_random(seed, device, _DTYPES[options.dtype])
        r = cls(model, options, device)
        r.config = cfg
        return r

    def _build_caches(self) -> None:
        """Sizes and allocates what the run entries keep between steps. Every question about a cache is put to its
        CacheSpec (group, bytes a page, bytes a request, tensors), so a mixer may bring a kind of its own."""
        opt = self.options
        needs = self.model.cache_needs()
        self.max_blocks_per_seq = -(-opt.max_model_len // self.page_size)
        # one more slot than requests: the padded rows of a replayed graph read and write the spare
        self.num_slots = opt.max_num_seqs + 1
        # groups: run entries whose paged needs coincide share block tables
        keys: list[tuple] = []
        windows: list = []
        entry_group: list[int | None] = []
        for need in needs:
            k = need.group_key() if need is not None else None
            if k is None:
                entry_group.append(None)
                continue
            if k not in keys:
                keys.append(k)
                windows.append(need.window)
            elif windows[keys.index(k)] != need.window:
                raise ValueError(f"cache group {k!r} is asked for with windows {windows[keys.index(k)]} and {need.window}: "
                                 "the group key must tell them apart")
            entry_group.append(keys.index(k))
        # prompt portions end where every layer's own chunks end: the user's alignment raised to what this model's
        # caches ask (kept here, for the scheduler of this runner: the options object may serve another model too)
        import math
        self.chunk_alignment = int(opt.prefill_chunk_alignment or 1)
        for n in needs:
            if n is not None and n.chunk_alignment > 1:
                self.chunk_alignment = math.lcm(self.chunk_alignment, n.chunk_alignment)
        page_bytes = sum(n.page_bytes(self.page_size, self.dtype) for n in needs if n is not None)
        slot_bytes = sum(n.slot_bytes(self.dtype) for n in needs if n is not None) * self.num_slots
        if opt.num_blocks is not None:
            num_blocks = opt.num_blocks
        else:
            # weights and activation buffers are allocated; the cache takes what is left
            # (models/qwen3/src/model.rs:545-603): min(free, total * util - used) - reserve - logits
            free, total = torch.cuda.mem_get_info(self.device)
            used = total - free
            reserve = 512 << 20
            budget = min(free, int(total * opt.gpu_memory_utilization) - used) - reserve - slot_bytes
            budget -= 3 * self.max_rows * self.model.spec.vocab_size * 4
            num_blocks = budget // max(page_bytes, 1) if page_bytes else 1
            if num_blocks <= 0:
                raise RuntimeError("no memory is left for the cache after weights and buffers")
        if keys and self.max_blocks_per_seq > num_blocks:
            raise RuntimeError(f"one request of max_model_len {opt.max_model_len} needs {self.max_blocks_per_seq} "
                               f"pages, the pool has {num_blocks}")
        self.num_blocks = int(num_blocks)
        self.group_specs = [GroupSpec(self.page_size, self.num_blocks, window=w) for w in windows]
        prefix = opt.enable_prefix_caching
        rebuilt_from_tokens = all(n.recomputable for n in needs if n is not None)
        if prefix is None:
            # reusing pages is only the whole truth where the pages are: no layer drops keys, none keeps state of its own
            prefix = bool(keys) and all(g.window is None for g in self.group_specs) and rebuilt_from_tokens
        elif prefix and not rebuilt_from_tokens:
            raise ValueError("the prefix cache cannot restore a layer's own state: switch it off for this model")
        self.cache = CacheManager(self.group_specs, opt.max_num_seqs, prefix_caching=prefix)
        self.cache_views: list[CacheView] = []
        self._slotted: list[tuple] = []     # (spec, tensors) of the entries with per-request memory
        own: dict[int, CacheView] = {}
        for i, (e, need) in enumerate(zip(self.model.run, needs)):
            if e.cache != i:
                src = own[e.cache]
                self.cache_views.append(CacheView(src.group, owner=False, tensors=src.tensors))
                continue
            if need is None:
                view = CacheView(None, owner=True)
            else:
                tensors = need.allocate(self.num_blocks, self.page_size, self.num_slots, self.dtype, self.device)
                view = CacheView(entry_group[i], owner=True, tensors=tensors)
                if need.slot_bytes(self.dtype) > 0:
                    self._slotted.append((need, tensors))
            own[i] = view
            self.cache_views.append(view)

    @property
    def state_tensors(self) -> list:
        """The per-request tensors of all entries that have any (what tests and reports look at)."""
        return [t for _, tensors in self._slotted for t in tensors.values()]

    def _reset_fresh_slots(self) -> None:
        fresh = self.cache.take_fresh_slots()
        if fresh and self._slotted:
            idx = torch.tensor(fresh, device=self.device, dtype=torch.long)
            for need, tensors in self._slotted:
                need.reset_slots(tensors, idx)

    def warm_up(self) -> None:
        """Runs one step of every row count that the library's products can meet, largest first, with made-up
        requests that are freed again, so that every shape has its algorithm (measured now, or read from the plan
        file) before the first real step; no later step times anything, and what a product computes does not
        depend on when its shape first came up. Nothing to do in 32-bit (own kernels only) or without measuring."""
        opt = self.options
        if self.dtype != torch.bfloat16 or opt.gemm_tuning != "measured" or not blaslt.available() or not self.group_specs:
            return
        most = min(self.max_tokens, self.num_blocks * self.page_size, opt.max_num_seqs * opt.max_model_len)
        sizes = sorted({min(t, most) for t in gemm.row_buckets(most) if t > gemm.SMALL_M}, reverse=True)
        met = blaslt.worth_measuring_met
        with blaslt.measuring():
            for n, total in enumerate(sizes):
                entries, left, i = [], total, 0
                while left > 0:
                    take = min(left, opt.max_model_len)
                    rid = ("warm-up", i)
                    if not self.reserve(rid, 0, take):
                        self.finish(rid)
                        break
                    entries.append(Entry(rid, [0] * take, 0, []))
                    left -= take
                    i += 1
                if left == 0:
                    want, e = min(total, self.max_rows), 0
                    while want > 0:     # logits at as many rows as the head can be asked for
                        k = min(want, len(entries[e].tokens))
                        entries[e].want = list(range(k))
                        want -= k
                        e += 1
                    self.step(entries)
                for e in entries:
                    self.finish(e.req_id)
                if n == 0 and blaslt.worth_measuring_met == met:
                    break       # not even the largest step holds a product worth measuring: a small model
        torch.cuda.synchronize(self.device)

    # ---- the step function ---------------------------------------------------------------------
    def step(self, entries: list[Entry]) -> torch.Tensor:
        """Runs one batch. Pages for every entry's tokens must have been allocated.
        Returns float32 logits [sum(len(e.want)), vocab] in the order of entries and of want
        (a view of a buffer that the next step overwrites)."""
        single_rows = all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)
        return self._run(len(entries), single_rows, lambda pad: self.batch.fill(entries, self.cache, pad_to=pad))

    def step_planned(self, scheduler, plan, greedy: bool = False) -> torch.Tensor:
        """The same step function for the step a scheduler has just planned: the batch is written
        straight from the tokens and tables the host core holds. Logits come back for the
        requests of the plan that sample, in the plan's order.
        greedy: every row will take its best token; a step that replays a graph then finds them itself
        (batch.last_tokens, `argmax_done` says so afterwards), one launch and one gap fewer after the graph."""
        return self._run(len(plan), plan.single_rows_that_sample,
                         lambda pad: self.batch.fill_planned(scheduler, pad_to=pad), greedy)

    def _run(self, n: int, single_rows: bool, fill, greedy: bool = False) -> torch.Tensor:
        timed = self.phases is not None
        if timed:
            import time
            self._began = time.perf_counter()
        self.argmax_done = False
        if self._graphs_allowed and single_rows and 0 < n <= self._buckets[-1]:
            out = self._graph_step(n, fill, greedy)
        elif self._portion_graphs_allowed and not single_rows:
            out = self._portion_step(fill)
        else:
            self._send(fill, None)
            self._reset_fresh_slots()
            out = self.model.forward(self.batch, self.cache_views)
        if timed:
            self._events[1].record()
            self.phases["launch"] += time.perf_counter() - self._began
        return out

    def _send(self, fill, pad, shape=None):
        """Writes the step into the pinned buffer and starts its copy to the device. While phases are measured
        (Engine.measure_phases) the host's time up to here counts as "fill", what follows as "launch", and two events
        bracket the step on the device. shape: called between the two, may pad the step; its result is returned."""
        fill(pad)
        shaped = shape() if shape is not None else None
        self.batch.upload()
        self._mark_sent()
        return shaped

    def _mark_sent(self) -> None:
        if self.phases is not None:
            import time
            now = time.perf_counter()
            self.phases["fill"] += now - self._began
            self._began = now
            self._events = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            self._events[0].record()

    def take_gpu_events(self):
        ev, self._events = self._events, None
        return ev

    def _graph_step(self, n: int, fill, greedy: bool = False) -> torch.Tensor:
        """A step of single rows replays a HIP graph captured for its batch-size bucket
        (crates/layers/src/exec.rs:83-222, models/qwen3/src/executor.rs:995-1014). All step
        inputs live at fixed addresses; what varies between replays is their content."""
        b = self.batch
        bucket = next(x for x in self._buckets if x >= n)
        self._send(fill, bucket)
        self._reset_fresh_slots()   # outside the graph: which slots are fresh changes from step to step
        greedy = greedy and bucket <= b.last_tokens.numel()
        self.argmax_done = greedy
        g = self._graphs.get((bucket, greedy))
        if g is not None:
            g.replay()
            return self.model.logits[:n]
        # The first step of a bucket runs eagerly (first-use initialisation must not happen under capture) and its
        # result is the step's result; the capture that follows records the same launches without running them.
        # Nothing is replayed in this step: a part with state of its own must see each step once.
        def forward():
            logits = self.model.forward(b, self.cache_views)
            if greedy:      # (padded rows find a token as well; nobody reads it)
                if self._argmax_scratch is None:
                    self._argmax_scratch = ops.argmax_scratch(self.max_rows, logits.shape[1], self.device)
                ops.argmax(logits, b.last_tokens, bucket, self._argmax_scratch)

        forward()
        self._graphs[(bucket, greedy)] = self._capture(forward)
        return self.model.logits[:n]

    PORTION_GRAPH_AFTER = 2     # a step's counts must have come up this often before a graph is captured for them
    MAX_PORTION_GRAPHS = 96

    def _portion_shape(self):
        """Pads the step just filled up to counts that a graph can stand for, and makes the host-side facts parts
        choose kernels by a function of those counts alone. Returns (key, logits rows of the real requests), or None
        where the step stays as it is (and runs eagerly): it wants more rows than it has requests, or no padding fits.

        The counts: tokens up to the next row count the matrix products round to anyway (16 at most where the
        step has no more: the few-row products take other forms there), requests up to the next
        bucket of the decode graphs, one logits row a request (none if the step wants none), the longest portion up
        to the next power of two, and which of the three ways single rows are served (all of them are, some, none)."""
        b, opt = self.batch, self.options
        T, B, R = b.num_tokens, b.num_reqs, b.num_rows
        if R > B or B > self._buckets[-1]:
            return None
        later = [x for x in self._buckets if x >= B]
        Bp = Tp = None
        for cand in later:
            need = T + (cand - B)               # a made-up request brings a token at least
            # (up to 16 rows the products take the norms along: such a step stays one)
            tp = 16 if need <= 16 else gemm.row_bucket(need)
            if tp > T and cand == B:
                continue                        # made-up tokens need a made-up request
            Bp, Tp = cand, tp
            break
        if Bp is None or Tp > self.max_tokens or (R and Bp > self.max_rows):
            return None
        last = Tp - T - (Bp - B - 1) if Bp > B else 0         # tokens of the last made-up request
        if last > opt.max_model_len:
            return None
        real_rows = R
        b.pad(Bp, Tp, Bp if R else 0)
        q = b.max_q_len
        qp = min(Tp, max(16, 1 << (q - 1).bit_length()))
        route = 2 if b.num_singles == Bp else 1 if b.num_singles >= 4 else 0
        b.max_q_len, b.all_decode = qp, route == 2
        b.num_singles = Bp if route == 2 else 4 if route == 1 else 0
        return (Tp, Bp, b.num_rows, qp, route), real_rows

    def _portion_step(self, fill) -> torch.Tensor:
        """A step with prompt portions: eager the first times its counts come up, then captured, then replayed."""
        b = self.batch
        shaped = self._send(fill, None, self._portion_shape)
        self._reset_fresh_slots()
        if shaped is None:
            return self.model.forward(b, self.cache_views)
        key, rows = shaped
        g = self._portion_graphs.get(key)
        if g is not None:
            g.replay()
            self.portion_replays += 1
            return self.model.logits[:rows]
        self.model.forward(b, self.cache_views)
        seen = self._portion_seen[key] = self._portion_seen.get(key, 0) + 1
        if seen >= self.PORTION_GRAPH_AFTER and len(self._portion_graphs) < self.MAX_PORTION_GRAPHS:
            self._portion_graphs[key] = self._capture(lambda: self.model.forward(b, self.cache_views))
        return self.model.logits[:rows]

    def _capture(self, forward) -> torch.cuda.CUDAGraph:
        """Records forward()'s launches into a graph without running them (the step has run eagerly just before)."""
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        if self._capture_stream is None:
            self._capture_stream = torch.cuda.Stream(device=self.device)
        side = self._capture_stream
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            # by hand: torch's capture context would collect garbage and empty the allocator's cache first
            g.capture_begin(pool=self._graph_pool)
            try:
                forward()
            finally:
                g.capture_end()
        torch.cuda.current_stream().wait_stream(side)
        if self._graph_pool is None:
            self._graph_pool = g.pool()
        return g

    # ---- request bookkeeping shared by replay and tests ------------------------------------------
    def reserve(self, req_id, start: int, n: int) -> bool:
        """Admits the request if new and allocates pages for tokens [start, start + n)."""
        if not self.cache.has(req_id):
            self.cache.admit(req_id)
        return self.cache.allocate(req_id, start, n)

    def advance(self, req_id, num_computed: int) -> None:
        """After a step: gives back pages a window has passed."""
        self.cache.release_passed(req_id, num_computed)

    def finish(self, req_id) -> None:
        self.cache.free(req_id)
