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


class CacheSpec:
    """What one run entry keeps between steps, and how its memory is made. The engine sizes, groups and allocates
    every cache through these methods only, so a mixer with another kind of cache (one vector a token, unequal key
    and value widths, a layout of its own) brings a subclass and nothing in the engine changes.

    Paged memory: entries whose `group_key()` is equal share a pool of pages and one block table a request; a page id
    is valid in the tensors of every entry of the group. `page_bytes` says what one page of this entry takes, and
    `allocate` makes the tensors for `num_blocks` pages. Per-request memory of fixed size: `slot_bytes` a request,
    `allocate` makes room for `num_slots` requests (one of them is a spare that padded rows of a replayed graph use),
    `reset_slots` clears the slots of requests that have just been admitted.
    """
    window: int | None = None      # W: pages whose keys all lie more than W before the next token are given back
    recomputable: bool = True      # the contents follow from the request's tokens alone (pages may be shared and refilled)
    chunk_alignment: int = 1       # prompt portions that do not end the request must end at a multiple of this

    def group_key(self) -> tuple | None:
        """Hashable name of the page group; None if nothing here is paged."""
        return None

    def page_bytes(self, page_size: int, dtype) -> int:
        return 0

    def slot_bytes(self, dtype) -> int:
        return 0

    def allocate(self, num_blocks: int, page_size: int, num_slots: int, dtype, device) -> dict:
        """name -> tensor; the mixer finds them as attributes of its CacheView."""
        return {}

    def reset_slots(self, tensors: dict, slots) -> None:
        """slots: int64 tensor of request slots that start from nothing."""


def _element_size(dtype) -> int:
    import torch
    return torch.empty((), dtype=dtype).element_size()


@dataclass(frozen=True)
class KVSpec(CacheSpec):
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

    def page_bytes(self, page_size, dtype):
        return 2 * self.kv_heads * self.head_dim * page_size * _element_size(dtype)

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        import torch
        from ..kernels import ops
        geometry = (num_blocks, self.kv_heads, page_size, self.head_dim)
        return {"k": torch.empty(ops.k_cache_shape(*geometry), dtype=dtype, device=device),
                "v": torch.empty(ops.v_cache_shape(*geometry), dtype=dtype, device=device)}


@dataclass(frozen=True)
class StateSpec(CacheSpec):
    """Cache need of a mixer with per-request state of fixed size (shape per request). The state cannot be rebuilt
    from pages, so a model that has one gets no prefix cache."""
    shape: tuple
    dtype: str = "float32"
    recomputable = False

    def slot_bytes(self, dtype):
        import torch
        n = 1
        for s in self.shape:
            n *= s
        return n * _element_size(getattr(torch, self.dtype))

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        import torch
        return {"state": torch.zeros((num_slots, *self.shape), dtype=getattr(torch, self.dtype), device=device)}

    def reset_slots(self, tensors, slots):
        tensors["state"].index_fill_(0, slots, 0)


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
    # optional, each a PartSpec of STREAM_OPS: applied in place to the embeddings before the first layer (tensors of
    # its own under embed_name + "post.") and to the logits after the head (under head_name + "post.")
    embed_post: PartSpec | None = None
    logits_post: PartSpec | None = None
