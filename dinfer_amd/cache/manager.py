"""The cache manager: pages per group of layers, a block table per request and
group, and a slot of fixed size per request. The state lives in the C++ class
of csrc/host/cache_manager.hpp; this front names requests by any hashable id
and turns status codes into exceptions.

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

import ctypes
import itertools
from dataclasses import dataclass

from .. import native

_I32, _I64 = ctypes.c_int32, ctypes.c_int64


@dataclass(frozen=True)
class GroupSpec:
    """window None: every key of the request is kept. window W: the last W keys."""
    page_size: int
    num_blocks: int
    window: int | None = None


class _PoolView:
    """What tests and reports read of one group's pool."""

    def __init__(self, manager: "CacheManager", group: int):
        self._m, self._g = manager, group
        self.num_blocks = manager.groups[group].num_blocks

    @property
    def num_free(self) -> int:
        return self._m.num_free(self._g)

    def free_list(self) -> list[int]:
        out = (_I32 * self.num_blocks)()
        n = native.checked("dh_cache_free_list", self._m._h, self._g, out, self.num_blocks)
        return list(out[:n])


class CacheManager:
    def __init__(self, groups: list[GroupSpec], max_seqs: int, prefix_caching: bool = False):
        """prefix_caching: full pages are named after the tokens of the prefix they end (needs groups that
        keep every key, one page size); ``lookup`` and ``commit`` use the names."""
        self.groups = list(groups)
        self.prefix_caching = bool(prefix_caching)
        if len(self.groups) > native.MAX_GROUPS:
            raise ValueError(f"{len(self.groups)} cache groups; at most {native.MAX_GROUPS} are supported")
        n = len(self.groups)
        arr = lambda vals: (_I32 * max(n, 1))(*vals)
        self._h = native.created("dh_cache_create", n, arr([g.page_size for g in self.groups]),
                                 arr([g.num_blocks for g in self.groups]),
                                 arr([-1 if g.window is None else g.window for g in self.groups]), int(max_seqs),
                                 int(self.prefix_caching))
        self.max_seqs = max_seqs
        self.pools = [_PoolView(self, g) for g in range(n)]
        self._handles: dict = {}          # request id -> the number the core knows it by
        self._pinned: set = set()         # ids whose number outlives free() (a scheduler owns them)
        self._numbers = itertools.count(1)
        self._slots = (_I32 * max_seqs)()
        self._need = (_I32 * max(n, 1))()

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        try:
            if h:
                native.fn("dh_cache_destroy")(h)
        except Exception:  # the interpreter is shutting down: the process ends anyway
            pass

    # ---- request numbers -------------------------------------------------------------------------
    def handle(self, req_id, create: bool = False, pin: bool = False) -> int:
        h = self._handles.get(req_id)
        if h is None:
            if not create:
                raise KeyError(f"request {req_id!r} is not live")
            h = self._handles[req_id] = next(self._numbers)
        if pin:
            self._pinned.add(req_id)
        return h

    def forget(self, req_id) -> None:
        """Drops the number of a request that a scheduler owned (after it has finished)."""
        self._pinned.discard(req_id)
        self._handles.pop(req_id, None)

    # ---- requests ------------------------------------------------------------------------------
    def has(self, req_id) -> bool:
        h = self._handles.get(req_id)
        return h is not None and bool(native.fn("dh_cache_has")(self._h, h))

    def can_admit(self) -> bool:
        return bool(native.fn("dh_cache_can_admit")(self._h))

    def admit(self, req_id) -> int:
        """Registers a request and gives it a state slot. Raises if it is known or no slot is free."""
        if self.has(req_id):
            raise KeyError(f"request {req_id!r} is already live")
        fresh = req_id not in self._handles
        try:
            return native.checked("dh_cache_admit", self._h, self.handle(req_id, create=True))
        except Exception:
            if fresh:
                self._handles.pop(req_id, None)
            raise

    def take_fresh_slots(self) -> list[int]:
        n = native.checked("dh_cache_take_fresh_slots", self._h, self._slots, self.max_seqs)
        return list(self._slots[:n])

    def slot_of(self, req_id) -> int:
        return native.checked("dh_cache_slot_of", self._h, self.handle(req_id))

    def live_requests(self) -> list:
        out = (_I64 * self.max_seqs)()
        n = native.fn("dh_cache_live_requests")(self._h, out, self.max_seqs)
        by_number = {h: rid for rid, h in self._handles.items()}
        return [by_number[h] for h in out[:n]]

    # ---- pages ---------------------------------------------------------------------------------
    def pages_needed(self, req_id, num_computed: int, num_new: int) -> list[int]:
        """Per group, how many new pages the tokens [num_computed, num_computed + num_new) need."""
        native.checked("dh_cache_pages_needed", self._h, self.handle(req_id), num_computed, num_new, self._need)
        return list(self._need[:len(self.groups)])

    def allocate(self, req_id, num_computed: int, num_new: int) -> bool:
        """Pages for tokens [num_computed, num_computed + num_new) in every group, or nothing at all."""
        return bool(native.checked("dh_cache_allocate", self._h, self.handle(req_id), num_computed, num_new))

    def release_passed(self, req_id, num_computed: int) -> int:
        """After a step: frees the pages of window groups that the token at position
        num_computed and all later ones cannot see. Returns how many were freed."""
        return native.checked("dh_cache_release_passed", self._h, self.handle(req_id), num_computed)

    def free(self, req_id) -> None:
        """Gives back everything the request holds, the last page first, so the tail of a
        request is what the next allocation takes (kv/manager.rs:338-345)."""
        native.checked("dh_cache_free", self._h, self.handle(req_id))
        if req_id not in self._pinned:
            del self._handles[req_id]

    # ---- prefix cache --------------------------------------------------------------------------
    def lookup(self, req_id, tokens: list) -> int:
        """For an admitted request that holds no page yet: takes the cached pages that match the start of
        its tokens (never all of them: the last token is always computed). Returns the tokens covered."""
        arr = (_I32 * max(len(tokens), 1))(*tokens)
        got = native.fn("dh_cache_lookup")(self._h, self.handle(req_id), arr, len(tokens))
        if got < 0:
            raise native.error(int(got), f"request {req_id!r}: ")
        return int(got)

    def commit(self, req_id, tokens: list, num_computed: int) -> None:
        """After a step: names the pages that tokens[:num_computed] fill completely."""
        arr = (_I32 * max(len(tokens), 1))(*tokens)
        native.checked("dh_cache_commit", self._h, self.handle(req_id), arr, num_computed)

    # ---- views for the step --------------------------------------------------------------------
    def block_table(self, req_id, group: int) -> list[int]:
        cap = self.groups[group].num_blocks
        out = (_I32 * cap)()
        n = native.checked("dh_cache_block_table", self._h, self.handle(req_id), group, out, cap)
        if n > cap:  # more entries than pages: entries of pages given back stay in the table as -1
            out = (_I32 * n)()
            n = native.checked("dh_cache_block_table", self._h, self.handle(req_id), group, out, n)
        return list(out[:n])

    def slot_mapping(self, req_id, group: int, start: int, n: int) -> list[int]:
        """Cache slots (page * page_size + offset) of positions start .. start + n - 1."""
        out = (_I64 * max(n, 1))()
        native.checked("dh_cache_slot_mapping", self._h, self.handle(req_id), group, start, n, out,
                       context=f"request {req_id!r}: ")
        return list(out[:n])

    def num_free(self, group: int = 0) -> int:
        return native.checked("dh_cache_num_free", self._h, group)

    def check(self) -> None:
        """Invariants: no page lost, none held twice, every held page in exactly one table;
        no state slot lost or held twice; every live request of the core has a name here."""
        native.checked("dh_cache_check", self._h)
        self.live_requests()
