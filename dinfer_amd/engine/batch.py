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
  state_slots  [B]   int32  the request's fixed-size state slot (padded rows: the spare slot max_reqs)
  logits_rows  [R]   int32  rows of the flat batch whose logits are wanted
  feedback_src [T]   int32  -1, or: the token's id is not in input_ids but is the feedback_src-th of the tokens the
                            step before sampled (last_tokens, on the device): a step planned before that one ended

All of them live in one device allocation at fixed addresses and are filled by
one host-to-device copy from one pinned buffer (crates/layers/src/exec.rs:338-467),
so a step can be replayed as a captured graph.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from .. import native


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
                   ("state_slots", np.int32, (max_reqs,)), ("logits_rows", np.int32, (max(max_rows, 1),)),
                   ("feedback_src", np.int32, (max_tokens,))]
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
        self.feedback_src = d["feedback_src"]
        # the tokens the last step sampled, one per sampling request in the step's order: the sampler writes them here
        self.last_tokens = torch.zeros(max(max_rows, 1), dtype=torch.int32, device=device)
        self.slot_mapping = [d["slot_mapping%d" % g] for g in range(len(max_blocks))]
        self.block_table = [d["block_table%d" % g] for g in range(len(max_blocks))]
        # where the C++ core writes: addresses inside the pinned buffer
        self._buffers = native.BatchBuffers()
        bb = self._buffers
        bb.n_groups, bb.max_tokens, bb.max_reqs, bb.max_rows = len(max_blocks), max_tokens, max_reqs, max_rows
        for name in ("input_ids", "positions", "cu_seqlens", "seq_lens", "state_slots", "logits_rows", "feedback_src"):
            setattr(bb, name, self.h[name].ctypes.data)
        for g, mb in enumerate(max_blocks):
            bb.slot_mapping[g] = self.h["slot_mapping%d" % g].ctypes.data
            bb.block_table[g] = self.h["block_table%d" % g].ctypes.data
            bb.max_blocks[g] = mb
        self._facts = native.BatchFacts()
        # host-side facts of the current step
        self.num_tokens = self.num_reqs = self.num_rows = 0
        self.max_q_len = self.max_seq_len = self.num_singles = 0
        self.all_decode = False
        self.req_ids: list = []
        self._copied = torch.cuda.Event() if pin else None

    @property
    def q_lens(self) -> list[int]:
        """Tokens per request of the current step (padding rows included)."""
        return np.diff(self.h["cu_seqlens"][:self.num_reqs + 1]).tolist()

    def fill(self, entries: list[Entry], cache, pad_to: int | None = None) -> None:
        """Writes the step into the pinned buffer from the entries and the cache manager's tables
        (csrc/host/step_batch.hpp does the writing).

        pad_to: for a step of single rows that replays a captured graph of that many requests, the
        batch is filled up with requests of one token at position 0 that write no cache slot
        (slot -1) and read page 0, which always exists (crates/layers/src/exec.rs:388-426).
        Their logits rows are computed and ignored."""
        B = len(entries)
        if B == 0:
            raise ValueError("a step needs at least one request with at least one token")
        i32 = np.int32
        rids = np.array([cache.handle(e.req_id) for e in entries], dtype=np.int64)
        starts = np.array([e.start for e in entries], dtype=i32)
        counts = np.array([len(e.tokens) for e in entries], dtype=i32)
        want_counts = np.array([len(e.want) for e in entries], dtype=i32)
        tokens = np.array([t for e in entries for t in e.tokens] or [0], dtype=i32)
        wants = np.array([w for e in entries for w in e.want] or [0], dtype=i32)
        self._wait_for_upload()
        rc = native.fn("dh_batch_fill")(cache._h, self._buffers, B, rids.ctypes.data, starts.ctypes.data,
                                        counts.ctypes.data, tokens.ctypes.data, want_counts.ctypes.data,
                                        wants.ctypes.data, pad_to or 0, self._facts)
        if rc < 0:
            raise self._named(native.error(rc), [e.req_id for e in entries])
        self.req_ids = [e.req_id for e in entries]
        self._take_facts()

    def fill_planned(self, scheduler, pad_to: int | None = None) -> None:
        """The same for the step a scheduler has just planned, straight from the tokens it holds."""
        self._wait_for_upload()
        rc = native.fn("dh_sched_fill")(scheduler._h, self._buffers, pad_to or 0, self._facts)
        if rc < 0:
            raise self._named(native.error(rc), scheduler.planned_ids())
        self.req_ids = scheduler.planned_ids()
        self._take_facts()

    @staticmethod
    def _named(exc: Exception, ids: list) -> Exception:
        """The core names an entry by its index; say which request that is."""
        import re
        msg = re.sub(r"entry (\d+)", lambda m: f"request {ids[int(m.group(1))]!r}", str(exc.args[0]))
        return type(exc)(msg)

    def _wait_for_upload(self) -> None:
        if self._copied is not None:
            self._copied.synchronize()  # the last upload has read the pinned buffer

    def _take_facts(self) -> None:
        f = self._facts
        self.num_tokens, self.num_reqs, self.num_rows = f.num_tokens, f.num_reqs, f.num_rows
        self.max_q_len, self.max_seq_len, self.num_singles = f.max_q_len, f.max_seq_len, f.num_singles
        self.all_decode = f.num_singles == f.num_reqs

    def pad(self, reqs: int, tokens: int, rows: int) -> None:
        """After fill(): made-up requests that write nothing bring the step to these counts (csrc/host/step_batch.hpp,
        pad_batch), so that it has the launch shapes of a graph captured for them."""
        rc = native.fn("dh_batch_pad")(self._buffers, self._facts, reqs, tokens, rows)
        if rc < 0:
            raise native.error(rc)
        self._take_facts()

    def upload(self) -> None:
        self._dev.copy_(self._host, non_blocking=True)
        if self._copied is not None:
            self._copied.record()
