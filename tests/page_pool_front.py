"""A pool of cache pages on its own, for the tests of the C++ class in csrc/host/block_pool.hpp (the engine reaches
that class only through the cache manager, which holds one pool per group).

``allocate(n)`` is all-or-nothing and takes pages from the head of the free
list; ``free(ids)`` puts the pages back at the head in the order given, so pages
that were just given back are the next ones handed out (crates/core/src/kv/block_pool.rs:128-147,160-182).
This bare pool names no pages; inside the cache manager the same C++ class also keeps named pages of the prefix
cache at the tail of its list. A page is held by at most one owner; freeing a page that is not held raises.
"""
from __future__ import annotations

import ctypes

from dinfer_amd import native


class BlockPool:
    def __init__(self, num_blocks: int):
        self._h = native.created("dh_pool_create", int(num_blocks))
        self.num_blocks = num_blocks

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        try:
            if h:
                native.fn("dh_pool_destroy")(h)
        except Exception:  # the interpreter is shutting down: the process ends anyway
            pass

    @property
    def num_free(self) -> int:
        return native.fn("dh_pool_num_free")(self._h)

    def allocate(self, n: int) -> list[int] | None:
        """n pages, or None (and no change) if fewer than n are free."""
        out = (ctypes.c_int32 * max(n, 1))()
        if not native.checked("dh_pool_allocate", self._h, n, out):
            return None
        return list(out[:n])

    def free(self, ids) -> None:
        ids = list(ids)
        arr = (ctypes.c_int32 * max(len(ids), 1))(*ids)
        native.checked("dh_pool_free", self._h, arr, len(ids))

    def free_list(self) -> list[int]:
        out = (ctypes.c_int32 * self.num_blocks)()
        n = native.fn("dh_pool_free_list")(self._h, out, self.num_blocks)
        return list(out[:n])

    def is_held(self, b: int) -> bool:
        return bool(native.fn("dh_pool_is_held")(self._h, b))

    def check(self) -> None:
        """Every page is either free exactly once or held (never both, never neither)."""
        native.checked("dh_pool_check", self._h)
