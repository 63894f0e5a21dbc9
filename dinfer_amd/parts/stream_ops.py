"""What a model may do to its token embeddings before the first layer, or to its logits after the head
(ModelSpec.embed_post / logits_post): a class of STREAM_OPS with `forward(x, rows)`, in place on the first rows
of x ([rows, width]: the stream in the engine's dtype, or the float32 logits). The architecture of this
repository uses neither; a multiplied embedding or softly capped logits are a matter of the spec, not of
DecoderModel.
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part
from .registry import STREAM_OPS


@STREAM_OPS.register("scale_softcap")
class ScaleSoftcap(Part):
    """x *= scale, then x = softcap * tanh(x / softcap) where a cap is given. No tensors."""

    def __init__(self, width: int, scale: float = 1.0, softcap: float | None = None):
        if softcap is not None and not softcap > 0:
            raise ValueError(f"softcap must be positive, got {softcap}")
        self.width, self.scale, self.softcap = width, float(scale), softcap

    def forward(self, x, rows: int) -> None:
        ops.scale_softcap(x, rows, self.scale, self.softcap)
