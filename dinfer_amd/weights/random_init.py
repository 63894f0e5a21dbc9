"""Random-weights mode: writes a model folder (config.json, model.safetensors)
from a configuration and a seed.

Every tensor is drawn from its own generator seeded by (seed, tensor name), so
its values do not depend on the other tensors or on their order:
matrix and table weights N(0, 0.02), norm gains 1 + N(0, 0.1). Values are drawn
in float32 and stored in the requested dtype (bfloat16 by default).
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from ..parts.spec import TensorSpec
from .safetensors_io import write_safetensors

LINEAR_STD = 0.02
GAIN_STD = 0.1


def tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def draw(seed: int, name: str, spec: TensorSpec, dtype: torch.dtype) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed(tensor_seed(seed, name))
    if spec.integer:
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "linear":
        t = torch.randn(spec.shape, generator=g, dtype=torch.float32) * LINEAR_STD
    elif spec.init == "gain":
        t = 1.0 + torch.randn(spec.shape, generator=g, dtype=torch.float32) * GAIN_STD
    elif spec.init == "zeros":
        t = torch.zeros(spec.shape, dtype=torch.float32)
    elif spec.init == "ones":
        t = torch.ones(spec.shape, dtype=torch.float32)
    else:
        raise ValueError(f"tensor {name!r}: unknown init {spec.init!r}")
    return t.to(dtype)


def draw_on_device(seed: int, name: str, spec: TensorSpec, dtype: torch.dtype, device) -> torch.Tensor:
    """The same rule as draw() (one generator per tensor, seeded by (seed, name); the same distributions), drawn by
    the device's generator: for measurements at sizes where a file would only cost time. The device's generator is
    another algorithm than the host's, so the values are not those of a folder written with the same seed."""
    if spec.integer or spec.init in ("zeros", "ones"):
        return draw(seed, name, spec, dtype).to(device)
    g = torch.Generator(device=device)
    g.manual_seed(tensor_seed(seed, name))
    t = torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32)
    if spec.init == "linear":
        t *= LINEAR_STD
    elif spec.init == "gain":
        t = 1.0 + t * GAIN_STD
    else:
        raise ValueError(f"tensor {name!r}: unknown init {spec.init!r}")
    return t.to(dtype)


def write_random_model(config, out_dir: str | Path, seed: int = 0, dtype: str = "bfloat16") -> Path:
    """config: a typed configuration of a registered architecture. Returns the folder."""
    from ..config.registry import get_architecture
    from ..parts.model import expected_tensors

    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    arch = get_architecture(config.ARCHITECTURE)
    spec = arch.build_spec(config)
    tdt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    expected, _optional = expected_tensors(spec)
    tensors = {name: draw(seed, name, ts, tdt) for name, ts in expected.items()}
    cfg = config.to_dict()
    cfg.setdefault("architectures", [config.ARCHITECTURE])  # the key the registry chooses the model by
    cfg["torch_dtype"] = dtype
    (out / "config.json").write_text(json.dumps(cfg, indent=2))
    write_safetensors(out / "model.safetensors", tensors, metadata={"format": "pt", "seed": seed})
    return out
