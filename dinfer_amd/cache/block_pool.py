"""A pool of cache pages.

``allocate(n)`` is all-or-nothing and takes pages from the head of the free
list; ``free(ids)`` puts the pages back at the head in the order given, so pages
that were just given back are the next ones handed out (crates/core/src/kv/block_pool.rs:128-147,160-182;
this engine has no prefix cache, so there is no LRU tail).
A page is held by at most one owner; freeing a page that is not held raises.
"""
from __future__ import annotations

from collections import deque


class BlockPool:
    def __init__(self, num_blocks: int):
        if num_blocks <= 0:
            raise ValueError(f"a pool needs at least one page, got {num_blocks}")
        self.num_blocks = num_blocks
        self._free: deque[int] = deque(range(num_blocks))
        self._held = bytearray(num_blocks)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, n: int) -> list[int] | None:
        """n pages, or None (and no change) if fewer than n are free."""
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if n > len(self._free):
            return None
        out = [self._free.popleft() for _ in range(n)]
        for b in out:
            self._held[b] = 1
        return out

    def free(self, ids) -> None:
        ids = list(ids)
        for b in ids:
            if not (0 <= b < self.num_blocks) or not self._held[b]:
                raise RuntimeError(f"page {b} is freed but not held")
            self._held[b] = 0
        self._free.extendleft(reversed(ids))

    def free_list(self) -> list[int]:
        return list(self._free)

    def is_held(self, b: int) -> bool:
        return bool(self._held[b])

    def check(self) -> None:
        """Every page is either free exactly once or held (never both, never neither)."""
        free = list(self._free)
        if len(set(free)) != len(free):
            raise AssertionError("a page is on the free list twice")
        for b in range(self.num_blocks):
            if bool(self._held[b]) == (b in set(free)):
                raise AssertionError(f"page {b} is {'held and free' if self._held[b] else 'lost'}")
