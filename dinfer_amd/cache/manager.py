"""The cache manager: pages per group of layers, a block table per request and
group, and a slot of fixed size per request.

Groups. Layers whose caches have the same page geometry and the same need
("all keys" or "the last W keys") form a group. A group has its own pool of
pages and each request has one block table per group; a page id is valid in
every layer of its group (each layer has its own page tensors, indexed by the
same ids), as in the reference (models/qwen3/src/model.rs:604-612,
crates/core/src/kv/manager.rs:52-56).

Allocation follows crates/core/src/kv/manager.rs:203-281: before a step a
request asks for the pages its next ``num_new`` tokens need; the answer is
all-or-nothing over all groups. A decode token that stays inside its last page
allocates nothing.

Giving back. All pages and the slot when the request ends or is preempted
(sched/mod.rs:783-803,672-680). In a window group also, after each step, every
page whose keys all lie before the window of the request's next token; its
block-table entry becomes -1 and is never read again.

State slots (in the manner of crates/layers/src/exec.rs:253-333). Each live
request holds one index in [0, max_seqs) for its whole life. A slot handed out
is reported by ``take_fresh_slots`` so that the engine zero-fills its state
before the first step that uses it.
"""
from __future__ import annotations

from dataclasses import dataclass

from .block_pool import BlockPool


@dataclass(frozen=True)
class GroupSpec:
    """window None: every key of the request is kept. window W: the last W keys."""
    page_size: int
    num_blocks: int
    window: int | None = None


class _Req:
    __slots__ = ("tables", "num_tokens", "slot")

    def __init__(self, n_groups: int, slot: int):
        self.tables: list[list[int]] = [[] for _ in range(n_groups)]
        self.num_tokens = 0  # tokens for which pages have been allocated
        self.slot = slot


class CacheManager:
    def __init__(self, groups: list[GroupSpec], max_seqs: int):
        if max_seqs <= 0:
            raise ValueError("max_seqs must be positive")
        self.groups = list(groups)
        self.pools = [BlockPool(g.num_blocks) for g in self.groups]
        self.max_seqs = max_seqs
        self._free_slots = list(range(max_seqs - 1, -1, -1))
        self._fresh_slots: list[int] = []
        self._reqs: dict = {}

    # ---- requests ------------------------------------------------------------------------------
    def has(self, req_id) -> bool:
        return req_id in self._reqs

    def can_admit(self) -> bool:
        return bool(self._free_slots)

    def admit(self, req_id) -> int:
        """Registers a request and gives it a state slot. Raises if it is known or no slot is free."""
        if req_id in self._reqs:
            raise KeyError(f"request {req_id!r} is already live")
        if not self._free_slots:
            raise RuntimeError(f"all {self.max_seqs} request slots are taken")
        slot = self._free_slots.pop()
        self._fresh_slots.append(slot)
        self._reqs[req_id] = _Req(len(self.groups), slot)
        return slot

    def take_fresh_slots(self) -> list[int]:
        out, self._fresh_slots = self._fresh_slots, []
        return out

    def slot_of(self, req_id) -> int:
        return self._reqs[req_id].slot

    def live_requests(self) -> list:
        return list(self._reqs)

    # ---- pages ---------------------------------------------------------------------------------
    def _first_needed_page(self, g: GroupSpec, next_pos: int) -> int:
        """Index of the first page a token at next_pos (and later ones) can still read."""
        if g.window is None:
            return 0
        first_key = max(0, next_pos - g.window + 1)
        return first_key // g.page_size

    def pages_needed(self, req_id, num_computed: int, num_new: int) -> list[int]:
        """Per group, how many new pages the tokens [num_computed, num_computed + num_new) need."""
        r = self._reqs[req_id]
        end = num_computed + num_new
        need = []
        for g, tab in zip(self.groups, r.tables):
            want = -(-end // g.page_size)
            need.append(max(0, want - len(tab)))
        return need

    def allocate(self, req_id, num_computed: int, num_new: int) -> bool:
        """Pages for tokens [num_computed, num_computed + num_new) in every group, or nothing at all."""
        if num_new <= 0:
            raise ValueError("a step feeds at least one token per request")
        r = self._reqs[req_id]
        need = self.pages_needed(req_id, num_computed, num_new)
        if any(n > p.num_free for n, p in zip(need, self.pools)):
            return False
        for n, pool, tab in zip(need, self.pools, r.tables):
            tab.extend(pool.allocate(n))
        r.num_tokens = max(r.num_tokens, num_computed + num_new)
        return True

    def release_passed(self, req_id, num_computed: int) -> int:
        """After a step: frees the pages of window groups that the token at position
        num_computed and all later ones cannot see. Returns how many were freed."""
        r = self._reqs[req_id]
        n = 0
        for g, pool, tab in zip(self.groups, self.pools, r.tables):
            if g.window is None:
                continue
            first = min(self._first_needed_page(g, num_computed), len(tab))
            dead = [b for b in tab[:first] if b >= 0]
            if dead:
                pool.free(dead)
                n += len(dead)
                for i in range(first):
                    tab[i] = -1
        return n

    def free(self, req_id) -> None:
        """Gives back everything the request holds, the last page first, so the tail of a
        request is what the next allocation takes (kv/manager.rs:338-345)."""
        r = self._reqs.pop(req_id)
        for pool, tab in zip(self.pools, r.tables):
            pool.free([b for b in reversed(tab) if b >= 0])
        self._free_slots.append(r.slot)
        if r.slot in self._fresh_slots:
            self._fresh_slots.remove(r.slot)

    # ---- views for the step --------------------------------------------------------------------
    def block_table(self, req_id, group: int) -> list[int]:
        return self._reqs[req_id].tables[group]

    def slot_mapping(self, req_id, group: int, start: int, n: int) -> list[int]:
        """Cache slots (page * page_size + offset) of positions start .. start + n - 1."""
        tab = self._reqs[req_id].tables[group]
        ps = self.groups[group].page_size
        out = []
        for pos in range(start, start + n):
            b = tab[pos // ps]
            if b < 0:
                raise RuntimeError(f"request {req_id!r}: position {pos} lies in a page that was given back")
            out.append(b * ps + pos % ps)
        return out

    def num_free(self, group: int = 0) -> int:
        return self.pools[group].num_free

    def check(self) -> None:
        """Invariants: no page lost, none held twice, every held page in exactly one table."""
        for gi, pool in enumerate(self.pools):
            pool.check()
            seen = set()
            for rid, r in self._reqs.items():
                for b in r.tables[gi]:
                    if b < 0:
                        continue
                    if b in seen:
                        raise AssertionError(f"group {gi}: page {b} is in two block tables")
                    if not pool.is_held(b):
                        raise AssertionError(f"group {gi}: page {b} of {rid!r} is on the free list")
                    seen.add(b)
            if len(seen) + pool.num_free != pool.num_blocks:
                raise AssertionError(f"group {gi}: {pool.num_blocks - pool.num_free - len(seen)} pages are lost")
        slots = [r.slot for r in self._reqs.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise AssertionError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_seqs:
            raise AssertionError("a state slot is lost")
