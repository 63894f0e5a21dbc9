"""Registries from a kind name to the class that implements it.

One registry per kind of part. A model is assembled only through these, so a
new mixer, feed-forward, norm, position encoding or block arrangement becomes
usable by registering a class; no file of the framework changes. STREAM_OPS holds what a
model may do to its embeddings before the first layer or to its logits after the head.
"""
from __future__ import annotations


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: dict[str, type] = {}

    def register(self, name: str, cls: type | None = None):
        """``REG.register("name", Cls)`` or as a decorator ``@REG.register("name")``."""
        def put(c):
            if name in self._items and self._items[name] is not c:
                raise KeyError(f"{self.what} {name!r} is already registered")
            self._items[name] = c
            return c
        return put if cls is None else put(cls)

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> type:
        try:
            return self._items[name]
        except KeyError:
            raise KeyError(f"unknown {self.what} {name!r}; known: {sorted(self._items)}") from None

    def names(self) -> list[str]:
        return sorted(self._items)

    def __contains__(self, name: str) -> bool:
        return name in self._items


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
STREAM_OPS = Registry("stream operation")
