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


def _i64(u: int) -> int:
    """The int64 with the bits of the uint64 u."""
    return u - (1 << 64) if u >= 1 << 63 else u


class Sampler:
    def __init__(self, device, max_rows: int, vocab: int):
        self.device, self.max_rows, self.vocab = device, max_rows, vocab
        self.out = torch.empty(max_rows, dtype=torch.int32, device=device)
        self.work: torch.Tensor | None = None  # [max_rows, vocab] float32, made on first non-greedy use

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
        if self.work is None:
            self.work = torch.empty((self.max_rows, self.vocab), dtype=torch.float32, device=self.device)
        dev = self.device
        f32 = lambda xs: torch.tensor(xs, dtype=torch.float32, device=dev)
        temperature = f32([p.temperature for p, *_ in rows])
        top_k = torch.tensor([p.top_k for p, *_ in rows], dtype=torch.int32, device=dev)
        top_p = f32([p.top_p for p, *_ in rows])
        min_p = f32([p.min_p for p, *_ in rows])
        seeds = torch.tensor([_i64(seed) for *_, seed in rows], dtype=torch.int64, device=dev)
        offsets = torch.tensor([n_out for _, n_out, *_ in rows], dtype=torch.int64, device=dev)
        ops.sample(logits, self.work, self.out, R, temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p,
                   seeds=seeds, offsets=offsets)
        return self.out[:R].tolist()

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
