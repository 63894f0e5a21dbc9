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


class Sampler:
    def __init__(self, device, max_rows: int, vocab: int):
        self.device, self.max_rows, self.vocab = device, max_rows, vocab
        self.out = torch.empty(max_rows, dtype=torch.int32, device=device)
        # made on first non-greedy use: [max_rows, vocab] float32 for rows that take the one-workgroup path,
        # the kernels' scratch, and the rows' options (filled in pinned host memory, copied once per step)
        self.work: torch.Tensor | None = None
        self.scratch: torch.Tensor | None = None
        self.rows_host: torch.Tensor | None = None
        self.rows_dev: torch.Tensor | None = None
        self.history: torch.Tensor | None = None   # [max_rows, vocab] int32, made on first use of a penalty
        self._slots: dict = {}                      # request -> [history slot, outputs already counted]
        self.phases: dict | None = None             # Engine.measure_phases: host time of the last launches and of the wait
        self._free: list = []

    def _buffers(self) -> None:
        if self.work is not None:
            return
        nbytes = self.max_rows * ops.SAMPLE_ROW.itemsize
        self.work = torch.empty((self.max_rows, self.vocab), dtype=torch.float32, device=self.device)
        self.scratch = torch.empty(ops.sample_scratch_bytes(self.max_rows, self.vocab), dtype=torch.uint8,
                                   device=self.device)
        self.rows_host = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
        self.rows_dev = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self._rows_np = self.rows_host.numpy().view(ops.SAMPLE_ROW)

    def sample(self, logits: torch.Tensor, rows: list) -> list[int]:
        """rows: per logits row (SamplingParams, num_output_tokens, prompt_ids, output_ids, seed[, request]).
        request: any hashable name of the request, under which its history is kept from step to step
        (forget() when it is over); without it a row with penalties sends its whole history every time."""
        R = len(rows)
        assert logits.shape[0] == R and R <= self.max_rows
        if R == 0:
            return []
        if all(p.is_greedy and not p.has_penalties for p, *_ in rows):
            if self.phases is not None:
                return self._timed(lambda: ops.argmax(logits, self.out, R), R)
            ops.argmax(logits, self.out, R)
            return self.out[:R].tolist()
        if any(p.has_penalties for p, *_ in rows):
            self._penalties(logits, rows)
        self._buffers()
        rec = self._rows_np
        for i, (p, n_out, _prompt, _output, seed, *_key) in enumerate(rows):
            rec[i] = (p.temperature, p.top_k, p.top_p, p.min_p, seed & 0xFFFFFFFFFFFFFFFF, n_out)
        n = R * ops.SAMPLE_ROW.itemsize
        # pinned memory the device may still be reading from the step before: this step's tokens were read
        # back (tolist) before it returned, so that copy is done
        self.rows_dev[:n].copy_(self.rows_host[:n], non_blocking=True)
        any_filter = any(p.top_k > 0 or p.top_p < 1.0 for p, *_ in rows)
        if self.phases is not None:
            return self._timed(lambda: ops.sample_rows(logits, self.work, self.scratch, self.rows_dev, self.out, R,
                                                       any_filter=any_filter), R)
        ops.sample_rows(logits, self.work, self.scratch, self.rows_dev, self.out, R, any_filter=any_filter)
        return self.out[:R].tolist()   # waits for the stream, and with it for the copy out of rows_host

    def _timed(self, launch, R: int) -> list[int]:
        """The last launches of sample() with the host's time split into issuing them and waiting for the tokens."""
        import time
        t0 = time.perf_counter()
        launch()
        t1 = time.perf_counter()
        tokens = self.out[:R].tolist()
        self.phases["sample"] += t1 - t0
        self.phases["wait"] += time.perf_counter() - t1
        return tokens

    def forget(self, key) -> None:
        """The request is over: its history slot is free again."""
        st = self._slots.pop(key, None)
        if st is not None:
            self._free.append(st[0])

    def _penalties(self, logits, rows) -> None:
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
                ops.history_add(self.history, torch.from_numpy(np.asarray(entries, dtype=np.int32)).to(self.device))
            ops.penalties_dense(logits, R, self.history, torch.from_numpy(pen.view(np.uint8)).to(self.device))
        finally:
            self._free += passing
