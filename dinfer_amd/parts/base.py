"""Interfaces of the parts a model is put together from.

Every part gets its sizes and constants as constructor parameters, lists the
tensors it wants from the weight file under local names, takes them in
``load``, reserves its activation buffers in ``bind`` and computes in
``forward``. No part knows which model it is in or which layer it is.
"""
from __future__ import annotations

from typing import Callable

import torch

from .spec import CacheSpec, TensorSpec


class Workspace:
    """Activation buffers [max_tokens, cols], shared by name between layers.

    Layers run one after the other, so two layers asking for the same
    (name, cols, dtype) get the same memory. Addresses never change after
    ``bind``, which lets a step be captured as a HIP graph.
    """

    def __init__(self, device, dtype: torch.dtype, max_tokens: int):
        self.device, self.dtype, self.max_tokens = device, dtype, max_tokens
        self._bufs: dict[tuple, torch.Tensor] = {}

    def buffer(self, name: str, cols: int, dtype: torch.dtype | None = None, rows: int | None = None) -> torch.Tensor:
        dt = dtype or self.dtype
        r = rows or self.max_tokens
        k = (name, cols, dt, r)
        b = self._bufs.get(k)
        if b is None:
            b = torch.empty((r, cols), dtype=dt, device=self.device)
            self._bufs[k] = b
        return b

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


class BuildContext:
    """What a part may know about the engine it is built into."""

    def __init__(self, device, dtype: torch.dtype, max_tokens: int, max_rows: int, page_size: int,
                 max_reqs: int = 1, max_seq_len: int | None = None):
        """max_tokens / max_rows / max_reqs: the largest step; max_seq_len: the longest request
        (None: unknown), for parts whose launch shapes are sized for it."""
        self.device, self.dtype = device, dtype
        self.max_tokens, self.max_rows, self.page_size, self.max_reqs = max_tokens, max_rows, page_size, max_reqs
        self.max_seq_len = max_seq_len
        self.workspace = Workspace(device, dtype, max_tokens)
        self._shared: dict = {}

    def share(self, key, make):
        """One object for all parts that ask under the same key (a table every layer would otherwise build for itself)."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]


class Part:
    # True: forward reads what changes from step to step from the batch's device tensors only (see Mixer.capturable)
    capturable = True
    # the same promise for steps with prompt portions (see Mixer.capturable_portions)
    capturable_portions = True

    def tensors(self) -> dict[str, TensorSpec]:
        """Local tensor name -> what the weight file must hold for it."""
        return {}

    def load(self, get: Callable[..., torch.Tensor]) -> None:
        """get(local_name, compute=False) returns the tensor on the device.
        compute=True asks for the engine's dtype (matrix-product operands)."""

    def bind(self, ctx: BuildContext) -> None:
        """Reserves buffers; called once before the first forward."""


class Norm(Part):
    def forward(self, x, out, n_rows: int, *, residual=None, rows=None):
        """out[r] = norm(x[src r]); with residual: residual = x + residual first, normed after."""
        raise NotImplementedError

    def carried(self):
        """(gain, offset, eps) if the norm is y = x / sqrt(mean(x^2) + eps) * (gain + offset), which the products
        around it can carry (see Carried); None for any other norm."""
        return None


class Carried:
    """A norm that is still to be applied to the residual stream, carried by the products around it: the product
    that completed the stream has left `xg` (the stream times the norm's gain) and `stats` (per row, `cols` partial
    sums of the squares of the stream); a product that takes xg as its operand and multiplies its result rows by
    rsqrt(sum(stats) / width + eps) has applied the norm. A consumer that cannot do that calls `materialise()`,
    which runs the norm's own kernel on the (complete) stream. Without xg (`scaled` False) the product has only
    added into the stream (steps of many rows), and `materialise()` is the one way on; `ready`: the product's last
    kernel has written the norm's output into `buf` already, and `materialise()` only hands it over."""
    __slots__ = ("xg", "stats", "cols", "eps", "width", "norm", "stream", "buf", "rows", "ready")

    def __init__(self, xg, stats, cols, eps, width, norm, stream, buf, rows, ready=False):
        self.xg, self.stats, self.cols, self.eps, self.width = xg, stats, cols, eps, width
        self.norm, self.stream, self.buf, self.rows, self.ready = norm, stream, buf, rows, ready

    @property
    def scaled(self) -> bool:
        return self.xg is not None

    def materialise(self) -> torch.Tensor:
        return self.buf if self.ready else self.norm.forward(self.stream, self.buf, self.rows)


class Into:
    """Where a part's last product may put its result instead of into a buffer of its own: added to `stream`
    in place, leaving a Carried for `norm`, the norm that reads the stream next (xg, stats, buf: the buffers for it).
    A part that cannot (sizes, dtype, a last operation that is no product) ignores it and returns its buffer."""
    __slots__ = ("stream", "norm", "xg", "stats", "buf")

    def __init__(self, stream, norm, xg, stats, buf):
        self.stream, self.norm, self.xg, self.stats, self.buf = stream, norm, xg, stats, buf


class PositionEncoding(Part):
    """How a mixer's queries and keys learn their positions. Two forms:

    fused (the default): a rotation of q and k by a table, which the mixer's kernel applies together with the per-head
    norm and the cache write: `table()` gives float32 [positions, rotary_dim] = [cos | sin] (None: no rotation),
    `rotary_dim` says how many leading dims of a head turn and `style` how they pair up.

    not fused (`fused = False`): anything else that acts on q and k: the mixer calls `transform(q, k, positions)`
    between the per-head norm and the cache write, so the keys in the cache carry it.
    """
    fused: bool = True
    rotary_dim: int = 0
    style: int = 0  # 0: pairs (i, i + rotary_dim/2); 1: pairs (2i, 2i+1)

    def table(self) -> torch.Tensor | None:
        return None

    def transform(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        """q [T, heads, D] and k [T, kv_heads, D]: views of the step's buffer, changed in place; positions int32 [T]
        on the device (read them there: a captured step is replayed with other contents)."""
        raise NotImplementedError


class CacheView:
    """The cache of one run entry as its mixer sees it.

    group: index of the page group (block tables, slot mappings in the batch), None if the entry has no pages;
    tensors: what the entry's CacheSpec allocated, by name, also reachable as attributes (an attention mixer reads
    `cache.k` and `cache.v`, a mixer with per-request state `cache.state`: [slots, *shape], indexed by
    batch.state_slots); owner: False if the memory belongs to another entry (read only).
    """

    def __init__(self, group: int | None = None, k=None, v=None, owner: bool = True, state=None, tensors: dict | None = None):
        self.group, self.owner = group, owner
        self.tensors = dict(tensors or {})
        for name, t in (("k", k), ("v", v), ("state", state)):
            if t is not None:
                self.tensors[name] = t

    def __getattr__(self, name):
        # only reached for names that are no attribute of the object: the cache's tensors, None for the usual
        # three where the entry has none of that kind
        tensors = self.__dict__.get("tensors", {})
        if name in tensors:
            return tensors[name]
        if name in ("k", "v", "state"):
            return None
        raise AttributeError(name)


class Mixer(Part):
    # True: forward also takes a Carried as x and the keyword `into` (an Into or None), and may return a Carried
    # when it has added its result to the stream itself. Parts that leave it False are given plain tensors.
    carries_norms = False
    # True: forward reads what changes from step to step (tokens, positions, slots, tables, lengths) from the batch's
    # device tensors only, never from host copies, and allocates nothing whose address must survive, so a step of
    # single rows captured once may be replayed for other requests. A mixer that leaves it False keeps every step of
    # its model eager.
    capturable = False
    # True: the promise of `capturable` also holds for steps that bring prompt portions, and whatever forward decides
    # on the host depends on batch.num_tokens, num_reqs, num_rows, max_q_len and num_singles alone (which such a
    # graph fixes: a step is padded up to them), never on the single requests' lengths (batch.q_lens and the like).
    # Then steps with portions whose counts come up again are replayed from graphs of their own.
    capturable_portions = False

    def cache_spec(self) -> CacheSpec | None:
        """What this mixer keeps between steps (a KVSpec, a StateSpec, a CacheSpec of its own), or None."""
        return None

    def forward(self, x: torch.Tensor, batch, cache: CacheView) -> torch.Tensor:
        """x [T, hidden] -> [T, hidden] (a workspace buffer; valid until the same part runs again)."""
        raise NotImplementedError


class FeedForward(Part):
    carries_norms = False   # as for Mixer

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """Arrangement of norm, mixer and feed-forward around the residual stream.

    forward(hidden, pending, batch, cache) -> pending': `hidden` is the residual
    stream, updated in place; `pending` is a branch output not yet added to it
    (None at the first layer). Deferring the add lets the next norm kernel do it.

    A block whose `input_norm()` is not None may be handed a Carried for that norm as `pending` (the
    stream is complete then); a block with `carries_norms` is told the next block's input norm as
    `next_norm` so that it can return one. Other blocks see neither.
    """
    carries_norms = False
    capturable = False   # an arrangement says so itself once all its parts are (see Mixer.capturable)
    capturable_portions = False

    def input_norm(self):
        """The norm this block applies to the stream first, if the block before may carry it; else None."""
        return None

    def forward(self, hidden, pending, batch, cache: CacheView):
        raise NotImplementedError
