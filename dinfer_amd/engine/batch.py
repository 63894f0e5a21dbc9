"""The flat batch of one step and its fixed device buffers.

A step holds, for each request in it, a contiguous run of its next tokens:
whole prompts, portions of prompts and single decoded tokens side by side
(crates/core/src/runner.rs:745-876). The fields and their rules:

  input_ids    [T]   int32  the tokens
  positions    [T]   int32  absolute position of each token
  slot_mapping [T]   int64  per cache group: page * page_size + position % page_size
  cu_seqlens   [B+1] int32  prefix sums of the tokens per request
  seq_lens     [B]   int32  request length after this step (start + n)
  block_table  [B, MB] int32 per cache group, -1 where no page is held
  state_slots  [B]   int32  the request's fixed-size state slot
  logits_rows  [R]   int32  rows of the flat batch whose logits are wanted

All of them live in one device allocation at fixed addresses and are filled by
one host-to-device copy from one pinned buffer (crates/layers/src/exec.rs:338-467),
so a step can be replayed as a captured graph.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class Entry:
    """One request's share of a step: its next tokens, where they start, which logits are wanted."""
    req_id: object
    tokens: list
    start: int
    want: list  # indices into `tokens`


class StepBatch:
    def __init__(self, device, max_tokens: int, max_reqs: int, max_rows: int, max_blocks: list[int]):
        self.device = device
        self.max_tokens, self.max_reqs, self.max_rows = max_tokens, max_reqs, max_rows
        self.max_blocks = list(max_blocks)
        layout = [("slot_mapping%d" % g, np.int64, (max_tokens,)) for g in range(len(max_blocks))]
        layout += [("input_ids", np.int32, (max_tokens,)), ("positions", np.int32, (max_tokens,)),
                   ("cu_seqlens", np.int32, (max_reqs + 1,)), ("seq_lens", np.int32, (max_reqs,)),
                   ("state_slots", np.int32, (max_reqs,)), ("logits_rows", np.int32, (max(max_rows, 1),))]
        layout += [("block_table%d" % g, np.int32, (max_reqs, mb)) for g, mb in enumerate(max_blocks)]
        off = 0
        spans = {}
        for name, dt, shape in layout:
            n = int(np.prod(shape)) * np.dtype(dt).itemsize
            spans[name] = (off, n, dt, shape)
            off += (n + 15) // 16 * 16
        self.nbytes = off
        pin = device.type == "cuda"
        self._host = torch.empty(off, dtype=torch.uint8, pin_memory=pin)
        self._dev = torch.empty(off, dtype=torch.uint8, device=device)
        hnp = self._host.numpy()
        tmap = {np.int32: torch.int32, np.int64: torch.int64}
        self.h, d = {}, {}
        for name, (o, n, dt, shape) in spans.items():
            self.h[name] = hnp[o:o + n].view(dt).reshape(shape)
            d[name] = self._dev[o:o + n].view(tmap[dt]).view(shape)
        self.input_ids, self.positions = d["input_ids"], d["positions"]
        self.cu_seqlens, self.seq_lens = d["cu_seqlens"], d["seq_lens"]
        self.state_slots, self.logits_rows = d["state_slots"], d["logits_rows"]
        self.slot_mapping = [d["slot_mapping%d" % g] for g in range(len(max_blocks))]
        self.block_table = [d["block_table%d" % g] for g in range(len(max_blocks))]
        # host-side facts of the current step
        self.num_tokens = self.num_reqs = self.num_rows = 0
        self.q_lens: list[int] = []
        self.starts: list[int] = []
        self.max_q_len = self.max_seq_len = 0
        self.all_decode = False
        self.max_len_bound = 0
        self.req_ids: list = []
        self.row_owner: list[tuple] = []  # (request index, token index) per logits row
        self._copied = torch.cuda.Event() if pin else None

    def fill(self, entries: list[Entry], cache, pad_to: int | None = None) -> None:
        """Writes the step into the pinned buffer from the entries and the cache manager's tables.

        pad_to: for a step of single rows that replays a captured graph of that many requests, the
        batch is filled up with requests of one token at position 0 that write no cache slot
        (slot -1) and read page 0, which always exists (crates/layers/src/exec.rs:388-426).
        Their logits rows are computed and ignored."""
        B = len(entries)
        T = sum(len(e.tokens) for e in entries)
        R = sum(len(e.want) for e in entries)
        if B == 0 or T == 0:
            raise ValueError("a step needs at least one request with at least one token")
        if B > self.max_reqs:
            raise ValueError(f"{B} requests in one step, the engine was built for {self.max_reqs}")
        if T > self.max_tokens:
            raise ValueError(f"{T} tokens in one step, the engine was built for {self.max_tokens}")
        if R > self.max_rows:
            raise ValueError(f"logits wanted at {R} places, the engine was built for {self.max_rows}")
        if self._copied is not None:
            self._copied.synchronize()  # the last upload has read the pinned buffer
        h = self.h
        t = r = 0
        self.q_lens, self.starts, self.req_ids, self.row_owner = [], [], [], []
        h["cu_seqlens"][0] = 0
        for g in range(len(self.max_blocks)):
            h["block_table%d" % g][:B].fill(-1)
        for b, e in enumerate(entries):
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.req_id!r} brings no token to this step")
            h["input_ids"][t:t + n] = e.tokens
            h["positions"][t:t + n] = np.arange(e.start, e.start + n, dtype=np.int32)
            for g, mb in enumerate(self.max_blocks):
                tab = cache.block_table(e.req_id, g)
                if len(tab) > mb:
                    raise ValueError(f"request {e.req_id!r} holds {len(tab)} pages, the block table has {mb} columns")
                h["block_table%d" % g][b, :len(tab)] = tab
                h["slot_mapping%d" % g][t:t + n] = cache.slot_mapping(e.req_id, g, e.start, n)
            h["cu_seqlens"][b + 1] = t + n
            h["seq_lens"][b] = e.start + n
            h["state_slots"][b] = cache.slot_of(e.req_id)
            for w in e.want:
                if not (0 <= w < n):
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {n} tokens")
                h["logits_rows"][r] = t + w
                self.row_owner.append((b, w))
                r += 1
            self.q_lens.append(n)
            self.starts.append(e.start)
            self.req_ids.append(e.req_id)
            t += n
        if pad_to is not None and pad_to > B:
            if T != B or R != B or pad_to > self.max_reqs or pad_to > self.max_tokens or pad_to > self.max_rows:
                raise ValueError("only a step of single rows that all want logits can be padded")
            P = pad_to
            h["input_ids"][B:P] = 0
            h["positions"][B:P] = 0
            h["cu_seqlens"][B + 1:P + 1] = np.arange(B + 1, P + 1, dtype=np.int32)
            h["seq_lens"][B:P] = 1
            h["state_slots"][B:P] = 0
            h["logits_rows"][B:P] = np.arange(B, P, dtype=np.int32)
            for g in range(len(self.max_blocks)):
                h["block_table%d" % g][B:P].fill(0)
                h["slot_mapping%d" % g][B:P] = -1
            self.q_lens += [1] * (P - B)
            self.starts += [0] * (P - B)
            T = B = R = P
        self.num_tokens, self.num_reqs, self.num_rows = T, B, R
        self.max_q_len = max(self.q_lens)
        self.max_seq_len = max(s + n for s, n in zip(self.starts, self.q_lens))
        self.all_decode = all(n == 1 for n in self.q_lens)
        # what kernels may assume about every seq_len of this step (a replayed graph fixes it to the model's limit)
        self.max_len_bound = self.max_seq_len

    def upload(self) -> None:
        self._dev.copy_(self._host, non_blocking=True)
        if self._copied is not None:
            self._copied.record()
