"""Descriptions from which a model is put together.

An architecture turns its configuration into a ``ModelSpec``: per layer the
kind and parameters of its mixer, feed-forward, norms and block arrangement,
plus the order in which layers run. Nothing here names a model; sizes and
constants arrive as parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class PartSpec:
    """Kind (a name in the matching registry) and constructor parameters of one part."""
    kind: str
    params: dict = field(default_factory=dict)

    def __hash__(self):
        return hash((self.kind, repr(sorted(self.params.items(), key=lambda kv: kv[0]))))


def part(kind: str, **params: Any) -> PartSpec:
    return PartSpec(kind, dict(params))


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part expects from the weight file.

    init: how the random-weights mode draws it: "linear" N(0, 0.02), "gain"
    1 + N(0, 0.1), "zeros", "ones". keep_f32: stays 32-bit even in a bfloat16
    engine when the file stores it so.
    """
    shape: tuple
    init: str = "linear"
    integer: bool = False


@dataclass(frozen=True)
class KVSpec:
    """Cache need of a mixer that stores a key and a value per token and kv head.

    window: None keeps every key of the request; W keeps the last W keys, so
    pages that the window has passed are given back while the request lives.
    """
    kv_heads: int
    head_dim: int
    window: int | None = None

    def group_key(self) -> tuple:
        # Layers of equal page geometry and equal window share block tables.
        return ("kv", self.kv_heads, self.head_dim, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Cache need of a mixer with per-request state of fixed size (shape per request)."""
    shape: tuple
    dtype: str = "float32"


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which block arrangement holds which mixer, feed-forward and norm.

    prefix: the layer's weight-name prefix; each part adds its own sub-prefix and
    local tensor names.
    """
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norm: PartSpec
    prefix: str


@dataclass(frozen=True)
class RunEntry:
    """One position in the execution order.

    layer: index into ModelSpec.layers (a layer may appear more than once: its
    weights are shared). cache: index of the run entry whose cache this entry
    uses; its own index by default. An entry that names another entry's cache
    reads it and writes nothing.
    """
    layer: int
    cache: int | None = None


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    layers: list  # [LayerSpec]
    run: list  # [RunEntry]
    final_norm: PartSpec
    final_norm_name: str
    embed_name: str
    head_name: str
    tie_embeddings: bool
    eos_token_ids: tuple = ()
