"""Turns logits rows into tokens on the device.

One row per request that reached the end of its known tokens. All rows greedy:
one argmax kernel. Otherwise: penalties (if any row has them; from a history of
each request's tokens kept on the device) and the chain temperature -> min_p ->
top-k/top-p -> draw, a row spread over many workgroups. A row's random number comes
from (seed, number of tokens the request has produced so far), so it does not
depend on the row's place in the batch or on the other rows
(crates/core/src/sampler.rs:1-4,84,197-212; models/qwen3/src/executor.rs:534-605).
"""
from __future__ import annotations

import numpy as np
import torch

from ..kernels import ops
from .params import MAX_LOGPROBS, TokenLogprobs


class Sampled:
    """The tokens of one launch(): on their way to pinned host memory until tokens() has waited for them."""

    def __init__(self, sampler, n: int, host, event, asked=None, about=None):
        self._sampler, self._n, self._host, self._event = sampler, n, host, event
        self._asked, self._about = asked, about     # per row k or None; the pinned (ids, logprobs, rank) of the launch

    def logprobs(self) -> list:
        """Per row None, or the TokenLogprobs of its token (rows whose request asked for them)."""
        if self._asked is None:
            return [None] * self._n
        self._event.synchronize()
        ids, lps, rank = self._about
        out: list = []
        for r, k in enumerate(self._asked):
            if k is None:
                out.append(None)
                continue
            i, l = ids[r, :k + 1].tolist(), lps[r, :k + 1].tolist()
            out.append(TokenLogprobs(i[0], l[0], int(rank[r]), list(zip(i[1:], l[1:]))))
        return out

    def tokens(self) -> list[int]:
        if self._n == 0:
            return []
        ph = self._sampler.phases
        if ph is None:
            self._event.synchronize()
        else:
            import time
            t0 = time.perf_counter()
            self._event.synchronize()
            ph["wait"] += time.perf_counter() - t0     # what the host stands still for
        return self._host[:self._n].tolist()


class Sampler:
    def __init__(self, device, max_rows: int, vocab: int, out: torch.Tensor | None = None, max_judged: int | None = None):
        """max_rows: the most rows a launch samples. out: int32 [>= max_rows] on the device where the sampled tokens
        are to land (the engine names the buffer that the next step may take its input tokens from); made here if
        absent. max_judged: the most rows about_rows() is asked about at once (default: max_rows)."""
        self.device, self.max_rows, self.vocab = device, max_rows, vocab
        self.max_judged = max(max_rows, max_judged or 0)
        self.out = out if out is not None else torch.empty(max_rows, dtype=torch.int32, device=device)
        assert self.out.dtype == torch.int32 and self.out.numel() >= max_rows
        # two launches may be in flight (a step planned ahead of the one that runs): what the host fills or reads
        # alternates between two pinned buffers (made at the first launch)
        self._tokens_host: list | None = None
        self._arg_scratch: torch.Tensor | None = None    # the argmax kernels' own memory between their two launches
        self._read: list | None = None
        self._turn = 0
        # made on first non-greedy use: [max_rows, vocab] float32 for rows that take the one-workgroup path,
        # the kernels' scratch, and the rows' options (filled in pinned host memory, copied once per launch)
        self.work: torch.Tensor | None = None
        self.scratch: torch.Tensor | None = None
        self.rows_host: list | None = None
        self.rows_dev: torch.Tensor | None = None
        self.history: torch.Tensor | None = None   # [max_rows, vocab] int32, made on first use of a penalty
        self._slots: dict = {}                      # request -> [history slot, outputs already counted]
        self.phases: dict | None = None             # Engine.measure_phases: host time of the last launches and of the wait
        self._free: list = []
        # made on first use of logprobs: a copy of the logits as the model gave them (where a bias or a penalty
        # changes them before the token is chosen), the kernel's outputs and their pinned landing places
        self._raw: torch.Tensor | None = None
        self._about_dev: tuple | None = None
        self._about_host: list | None = None
        self._given: list | None = None             # about_rows(): the tokens to judge, pinned, two turns
        self._given_dev: torch.Tensor | None = None
        self._given_read: list | None = None
        self._given_turn = 0
        self._arena: list | None = None             # per turn: [pinned bytes, bytes used, outgrown arenas still in flight]

    def _buffers(self) -> None:
        if self.work is not None:
            return
        nbytes = self.max_rows * ops.SAMPLE_ROW.itemsize
        self.work = torch.empty((self.max_rows, self.vocab), dtype=torch.float32, device=self.device)
        self.scratch = torch.empty(ops.sample_scratch_bytes(self.max_rows, self.vocab), dtype=torch.uint8,
                                   device=self.device)
        self.rows_host = [torch.empty(nbytes, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self.rows_dev = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self._rows_np = [h.numpy().view(ops.SAMPLE_ROW) for h in self.rows_host]

    def sample(self, logits: torch.Tensor, rows: list) -> list[int]:
        """launch() and the wait for its tokens in one."""
        return self.launch(logits, rows).tokens()

    def launch(self, logits: torch.Tensor, rows: list, done: bool = False) -> Sampled:
        """Issues the sampling of one token per logits row and the copy of the tokens to the host; returns at once.
        rows: per logits row (SamplingParams, num_output_tokens, prompt_ids, output_ids, seed[, request]).
        request: any hashable name of the request, under which its history is kept from step to step
        (forget() when it is over); without it a row with penalties sends its whole history every time.
        done: the tokens are in `out` already (every row is greedy and the step found them itself).
        At most two launches may be waiting for their tokens() at a time."""
        import time
        R = len(rows)
        assert logits.shape[0] == R and R <= self.max_rows
        if R == 0:
            return Sampled(self, 0, None, None)
        t0 = time.perf_counter() if self.phases is not None else None
        if self._tokens_host is None:
            self._tokens_host = [torch.empty(self.max_rows, dtype=torch.int32, pin_memory=True) for _ in range(2)]
            self._read = [torch.cuda.Event(), torch.cuda.Event()]
        turn = self._turn
        self._turn ^= 1
        asked = [p.logprobs for p, *_ in rows]
        if all(k is None for k in asked):
            asked = None
        changed = any(p.logit_bias or p.has_penalties for p, *_ in rows)
        given = logits                      # the logits as the model gave them
        if asked is not None and changed:
            if self._raw is None:
                self._raw = torch.empty((self.max_rows, self.vocab), dtype=torch.float32, device=self.device)
            given = self._raw
            given[:R].copy_(logits[:R])
        if all(p.picks_largest_logit for p, *_ in rows):
            if not done:
                if self._arg_scratch is None:
                    self._arg_scratch = ops.argmax_scratch(self.max_rows, self.vocab, self.device)
                ops.argmax(logits, self.out, R, self._arg_scratch)
        else:
            assert not done
            if self._arena is not None:
                self._arena[turn][1], self._arena[turn][2] = 0, []
            if any(p.logit_bias for p, *_ in rows):         # before the penalties (sampling.cu:286)
                self._bias(logits, rows, turn)
            if any(p.has_penalties for p, *_ in rows):
                self._penalties(logits, rows, turn)
            self._buffers()
            rec = self._rows_np[turn]
            for i, (p, n_out, _prompt, _output, seed, *_key) in enumerate(rows):
                rec[i] = (p.temperature, p.top_k, p.top_p, p.min_p, seed & 0xFFFFFFFFFFFFFFFF, n_out)
            n = R * ops.SAMPLE_ROW.itemsize
            # (the pinned buffer of this turn was last read by the launch before the last, whose tokens have been
            # waited for since)
            self.rows_dev[:n].copy_(self.rows_host[turn][:n], non_blocking=True)
            any_filter = any(p.top_k > 0 or p.top_p < 1.0 for p, *_ in rows)
            ops.sample_rows(logits, self.work, self.scratch, self.rows_dev, self.out, R, any_filter=any_filter)
        host = self._tokens_host[turn]
        host[:R].copy_(self.out[:R], non_blocking=True)
        about = self._logprobs(given, asked, R, turn) if asked is not None else None
        self._read[turn].record()
        if t0 is not None:
            self.phases["sample"] += time.perf_counter() - t0
        return Sampled(self, R, host, self._read[turn], asked, about)

    def about_rows(self, logits: torch.Tensor, targets: list, asked: list) -> Sampled:
        """The log-probabilities of given tokens: row r of logits is judged as if targets[r] had been chosen there,
        with its asked[r] most probable tokens beside it (the prompt's own tokens, each given the tokens before it:
        SamplingParams.prompt_logprobs). Returns at once; logprobs() of what comes back waits. At most two of these
        may be waiting at a time."""
        R = len(targets)
        assert logits.shape[0] == R == len(asked) and R <= self.max_judged and all(k is not None for k in asked)
        if R == 0:
            return Sampled(self, 0, None, None)
        if self._given is None:
            self._given = [torch.empty(self.max_judged, dtype=torch.int32, pin_memory=True) for _ in range(2)]
            self._given_dev = torch.empty(self.max_judged, dtype=torch.int32, device=self.device)
            self._given_read = [torch.cuda.Event(), torch.cuda.Event()]
        turn = self._given_turn
        self._given_turn ^= 1
        host = self._given[turn]
        host[:R] = torch.tensor(targets, dtype=torch.int32)
        self._given_dev[:R].copy_(host[:R], non_blocking=True)
        about = self._logprobs(logits, asked, R, 2 + turn, chosen=self._given_dev)
        self._given_read[turn].record()
        return Sampled(self, R, host, self._given_read[turn], asked, about)

    def _staged(self, turn: int, arr: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
        """arr on the device, sent through this turn's pinned arena without the host waiting for the stream (a copy
        from pageable memory would wait for the kernels of the step before, and a step launched ahead would no longer
        overlap with it). The arena of a turn was last read by the launch before the last, whose tokens have been
        waited for since; one that has to grow is kept until the turn comes round again."""
        if self._arena is None:
            self._arena = [[torch.empty(1 << 16, dtype=torch.uint8, pin_memory=True), 0, []] for _ in range(2)]
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        a = self._arena[turn]
        start = (a[1] + 15) & ~15
        if start + raw.size > a[0].numel():
            a[2].append(a[0])
            a[0], start = torch.empty(max(2 * a[0].numel(), raw.size), dtype=torch.uint8, pin_memory=True), 0
        a[0].numpy()[start:start + raw.size] = raw
        a[1] = start + raw.size
        dev = torch.empty(raw.size, dtype=torch.uint8, device=self.device)
        dev.copy_(a[0][start:start + raw.size], non_blocking=True)
        return dev.view(dtype).view(arr.shape)

    def _bias(self, logits, rows, turn: int) -> None:
        entries = [(i, t, b) for i, (p, *_rest) in enumerate(rows) for t, b in p.logit_bias.items() if t < self.vocab]
        if not entries:
            return
        where = self._staged(turn, np.array([(i, t) for i, t, _ in entries], dtype=np.int32), torch.int32)
        what = self._staged(turn, np.array([b for *_, b in entries], dtype=np.float32), torch.float32)
        ops.logit_bias(logits, len(rows), where, what)

    def _logprobs(self, given, asked, R: int, turn: int, chosen=None) -> tuple:
        """Issues the kernel that reads the tokens just chosen (self.out, or `chosen`) and the copies of what it
        found to pinned buffers (turn 0 and 1: launch()'s, 2 and 3: about_rows()'s); returns those (valid once the
        caller's event has passed)."""
        stride = MAX_LOGPROBS + 1
        if self._about_dev is None:
            dev, n = dict(device=self.device), self.max_judged
            self._about_dev = (torch.empty(n, dtype=torch.int32, **dev),                # k per row
                               torch.empty((n, stride), dtype=torch.int32, **dev),
                               torch.empty((n, stride), dtype=torch.float32, **dev),
                               torch.empty(n, dtype=torch.int32, **dev))
            self._about_host = [(torch.empty(n, dtype=torch.int32, pin_memory=True),
                                 torch.empty((n, stride), dtype=torch.int32, pin_memory=True),
                                 torch.empty((n, stride), dtype=torch.float32, pin_memory=True),
                                 torch.empty(n, dtype=torch.int32, pin_memory=True)) for _ in range(4)]
        k_dev, ids_dev, lp_dev, rank_dev = self._about_dev
        k_host, ids_host, lp_host, rank_host = self._about_host[turn]
        k_host[:R] = torch.tensor([-1 if k is None else k for k in asked], dtype=torch.int32)
        k_dev[:R].copy_(k_host[:R], non_blocking=True)
        ops.logprobs(given, self.out if chosen is None else chosen, k_dev, ids_dev, lp_dev, rank_dev, R)
        ids_host[:R].copy_(ids_dev[:R], non_blocking=True)
        lp_host[:R].copy_(lp_dev[:R], non_blocking=True)
        rank_host[:R].copy_(rank_dev[:R], non_blocking=True)
        return ids_host, lp_host, rank_host

    def forget(self, key) -> None:
        """The request is over: its history slot is free again."""
        st = self._slots.pop(key, None)
        if st is not None:
            self._free.append(st[0])

    def _penalties(self, logits, rows, turn: int) -> None:
        """Repetition, frequency and presence penalties, in place. The tokens a request has seen live on the
        device ([max_rows, vocab] int32, a slot per request with penalties); only what is new goes there:
        the distinct prompt tokens once, then the outputs since the last step."""
        if self.history is None:
            self.history = torch.empty((self.max_rows, self.vocab), dtype=torch.int32, device=self.device)
            self._free = list(range(self.max_rows - 1, -1, -1))
        R = len(rows)
        pen = np.zeros(R, dtype=ops.PENALTY_ROW)
        pen["slot"] = -1
        entries: list = []
        passing: list = []
        try:
            for i, (p, _n, prompt, output, _seed, *key) in enumerate(rows):
                if not p.has_penalties:
                    continue
                key = key[0] if key else None
                st = self._slots.get(key) if key is not None else None
                if st is None:
                    if not self._free:
                        raise RuntimeError(f"more than {self.max_rows} live requests with penalties")
                    st = [self._free.pop(), 0]
                    self.history[st[0]].zero_()
                    entries += [(st[0], t, 0) for t in set(prompt)]
                    if key is None:
                        passing.append(st[0])          # a row without a name: the slot lasts for this call
                    else:
                        self._slots[key] = st
                slot, counted = st
                entries += [(slot, t, 1) for t in output[counted:]]
                st[1] = len(output)
                pen[i] = (slot, p.repetition_penalty, p.frequency_penalty, p.presence_penalty)
            if entries:
                ops.history_add(self.history, self._staged(turn, np.asarray(entries, dtype=np.int32), torch.int32))
            ops.penalties_dense(logits, R, self.history, self._staged(turn, pen.view(np.uint8), torch.uint8))
        finally:
            self._free += passing
