"""Turns logits rows into tokens on the device.

One row per request that reached the end of its known tokens. All rows greedy:
one argmax kernel. Otherwise: penalties (if any row has them) and the fused
temperature -> min_p -> top-k/top-p -> draw kernel. A row's random number comes
from (seed, number of tokens the request has produced so far), so it does not
depend on the row's place in the batch or on the other rows
(crates/core/src/sampler.rs:1-4,84,197-212; models/qwen3/src/executor.rs:534-605).
"""
from __future__ import annotations

from collections import Counter

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams


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
        """rows: per logits row (SamplingParams, num_output_tokens, prompt_ids, output_ids, seed)."""
        R = len(rows)
        assert logits.shape[0] == R and R <= self.max_rows
        if R == 0:
            return []
        if all(p.is_greedy and not p.has_penalties for p, *_ in rows):
            ops.argmax(logits, self.out, R)
            return self.out[:R].tolist()
        if any(p.has_penalties for p, *_ in rows):
            self._penalties(logits, rows)
        self._buffers()
        rec = self._rows_np
        for i, (p, n_out, _prompt, _output, seed) in enumerate(rows):
            rec[i] = (p.temperature, p.top_k, p.top_p, p.min_p, seed & 0xFFFFFFFFFFFFFFFF, n_out)
        n = R * ops.SAMPLE_ROW.itemsize
        self.rows_dev[:n].copy_(self.rows_host[:n], non_blocking=True)
        any_filter = any(p.top_k > 0 or p.top_p < 1.0 for p, *_ in rows)
        ops.sample_rows(logits, self.work, self.scratch, self.rows_dev, self.out, R, any_filter=any_filter)
        return self.out[:R].tolist()   # waits for the stream, and with it for the copy out of rows_host

    def _penalties(self, logits, rows) -> None:
        ids, cnts, offs = [], [], [0]
        for p, _n, prompt, output, _s in rows:
            if p.has_penalties:
                c_out = Counter(output)
                seen = set(prompt) | set(output)
                for t in seen:
                    ids.append(t)
                    cnts.append(c_out.get(t, 0))
            offs.append(len(ids))
        dev = self.device
        i32 = lambda xs: torch.tensor(np.asarray(xs, dtype=np.int32), dtype=torch.int32, device=dev)
        f32 = lambda xs: torch.tensor(xs, dtype=torch.float32, device=dev)
        ops.penalties(logits, len(rows), i32(ids if ids else [0]), i32(cnts if cnts else [0]), i32(offs),
                      f32([p.repetition_penalty for p, *_ in rows]), f32([p.frequency_penalty for p, *_ in rows]),
                      f32([p.presence_penalty for p, *_ in rows]))
