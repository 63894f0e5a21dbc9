"""Loading a model's tensors by name, with one error for everything that is wrong.

The model says which tensors it expects (name -> TensorSpec). ``check`` compares
that list with the file's index and raises a single ``WeightError`` listing
missing tensors, unexpected tensors and wrong shapes together. ``fetch`` then
brings one tensor to the device:

  * stored BF16 / F16 -> the engine's dtype (bfloat16, or float32 on the 32-bit path),
  * stored F32 stays float32 unless the caller asks for the compute dtype
    (matrix-product weights run in the engine's dtype; gains and other small
    parameters keep their 32 bits),
  * integer tables -> int32.

Classes of error follow the reference, crates/layers/src/weights.rs:143,169-205,210
(missing tensor, size mismatch, unsupported dtype).
"""
from __future__ import annotations

import torch

from ..parts.spec import TensorSpec
from .safetensors_io import SafetensorsDir


class WeightError(ValueError):
    """Missing, unexpected or wrongly shaped tensors; the message lists all of them."""

    def __init__(self, missing, unexpected, wrong_shape, other=()):
        self.missing, self.unexpected, self.wrong_shape, self.other = list(missing), list(unexpected), list(wrong_shape), list(other)
        parts = []
        if self.missing:
            parts.append("missing tensors: " + ", ".join(self.missing))
        if self.unexpected:
            parts.append("unexpected tensors: " + ", ".join(self.unexpected))
        if self.wrong_shape:
            parts.append("wrong shapes: " + "; ".join(f"{n} is {list(got)}, expected {list(want)}"
                                                      for n, got, want in self.wrong_shape))
        if self.other:
            parts.append("; ".join(self.other))
        super().__init__("weights do not fit the model: " + " | ".join(parts))


class WeightLoader:
    def __init__(self, model_dir, device, dtype: torch.dtype):
        self.src = SafetensorsDir(model_dir)
        self.device = device
        self.dtype = dtype

    def check(self, expected: dict[str, TensorSpec], optional: set[str] = frozenset()) -> None:
        have = set(self.src.names())
        missing = sorted(n for n in expected if n not in have and n not in optional)
        unexpected = sorted(n for n in have if n not in expected and n not in optional)
        wrong, other = [], []
        for n, spec in expected.items():
            if n in have:
                ti = self.src.info(n)
                if tuple(ti.shape) != tuple(spec.shape):
                    wrong.append((n, ti.shape, spec.shape))
                is_int = ti.dtype_name.startswith(("I", "U", "BOOL"))
                if is_int != bool(spec.integer):
                    other.append(f"{n} is stored as {ti.dtype_name}, expected "
                                 f"{'an integer' if spec.integer else 'a floating-point'} tensor")
        if missing or unexpected or wrong or other:
            raise WeightError(missing, unexpected, wrong, other)

    def has(self, name: str) -> bool:
        return name in self.src

    def fetch(self, name: str, *, compute: bool = False) -> torch.Tensor:
        """compute=True: a matrix-product operand, always brought to the engine's dtype."""
        if name not in self.src:
            raise WeightError([name], [], [])
        t = self.src.read_to(name, self.device)   # conversions happen where the tensor lives
        if t.dtype in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool):
            return t.to(torch.int32)
        if t.dtype == torch.float64:
            t = t.to(torch.float32)
        if compute or t.dtype != torch.float32:
            t = t.to(self.dtype)
        return t.contiguous()

    def close(self) -> None:
        self.src.close()
