"""Reading and writing the safetensors container, by tensor name.

Format (as the reference's own parser reads it, crates/layers/src/weights.rs:1-4,
96-129): 8 bytes little-endian header length N, N bytes of JSON
``{name: {"dtype", "shape", "data_offsets": [start, end]}, "__metadata__": ...}``,
then the data; offsets count from byte 8 + N. Every ``*.safetensors`` file of a
folder is opened, sorted by name, into one index (weights.rs:79-88). Files are
memory-mapped; a tensor is materialised only when it is asked for.
"""
from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path

import torch

DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
NAMES = {v[0]: k for k, v in DTYPES.items()}


class WeightFileError(ValueError):
    pass


class TensorInfo:
    __slots__ = ("name", "dtype_name", "shape", "start", "end", "file")

    def __init__(self, name, dtype_name, shape, start, end, file):
        self.name, self.dtype_name, self.shape, self.start, self.end, self.file = name, dtype_name, shape, start, end, file


class _File:
    def __init__(self, path: Path):
        self.path = path
        self.fh = open(path, "rb")
        size = path.stat().st_size
        if size < 8:
            raise WeightFileError(f"{path}: too short for a safetensors header")
        # a private mapping: pages come from the page cache without a copy, and the buffer counts as writable, which
        # lets torch wrap it without complaint (nothing ever writes to it)
        self.mm = mmap.mmap(self.fh.fileno(), 0, access=mmap.ACCESS_COPY)
        (n,) = struct.unpack("<Q", self.mm[:8])
        if 8 + n > size:
            raise WeightFileError(f"{path}: header length {n} exceeds the file size {size}")
        try:
            self.header = json.loads(self.mm[8:8 + n].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not valid JSON: {e}") from e
        self.base = 8 + n
        self.size = size


class SafetensorsDir:
    """Index over all tensors of a model folder."""

    def __init__(self, model_dir: str | Path):
        d = Path(model_dir)
        paths = sorted(d.glob("*.safetensors"))
        if not paths:
            raise WeightFileError(f"no *.safetensors under {d}")
        self.files = [_File(p) for p in paths]
        self.index: dict[str, TensorInfo] = {}
        for f in self.files:
            for name, meta in f.header.items():
                if name == "__metadata__":
                    continue
                try:
                    dt, shape, (s, e) = meta["dtype"], tuple(int(x) for x in meta["shape"]), meta["data_offsets"]
                except (KeyError, TypeError, ValueError) as err:
                    raise WeightFileError(f"{f.path}: bad header entry for {name!r}: {err}") from err
                if dt not in DTYPES:
                    raise WeightFileError(f"{f.path}: tensor {name!r} has unsupported dtype {dt}")
                numel = 1
                for x in shape:
                    numel *= x
                if e - s != numel * DTYPES[dt][1] or s < 0 or f.base + e > f.size:
                    raise WeightFileError(f"{f.path}: tensor {name!r} has data range [{s}, {e}) that does not fit "
                                          f"its shape {shape} and dtype {dt} or the file")
                self.index[name] = TensorInfo(name, dt, shape, f.base + s, f.base + e, f)

    def names(self) -> list[str]:
        return sorted(self.index)

    def __contains__(self, name: str) -> bool:
        return name in self.index

    def info(self, name: str) -> TensorInfo:
        return self.index[name]

    def raw(self, name: str) -> torch.Tensor:
        """The tensor's bytes as a uint8 view of the mapped file: no copy. The view must be dropped before
        close(); callers copy it (to the device, or clone) right away."""
        ti = self.index[name]
        if ti.end == ti.start:
            return torch.empty(0, dtype=torch.uint8)
        return torch.frombuffer(ti.file.mm, dtype=torch.uint8, count=ti.end - ti.start, offset=ti.start)

    def read(self, name: str) -> torch.Tensor:
        """The tensor as stored (a CPU copy of its own, in its stored dtype)."""
        ti = self.index[name]
        dt, _ = DTYPES[ti.dtype_name]
        return self.raw(name).clone().view(dt).reshape(ti.shape)

    def read_to(self, name: str, device) -> torch.Tensor:
        """The tensor as stored, on `device`: one copy, from the mapped file straight to where it will live
        (the bytes are reinterpreted there, where the allocation is aligned whatever the file's offsets)."""
        ti = self.index[name]
        dt, _ = DTYPES[ti.dtype_name]
        raw = self.raw(name)
        dev = torch.device(device)
        moved = raw.clone() if dev.type == "cpu" else raw.to(dev)
        return moved.view(dt).reshape(ti.shape)

    def close(self) -> None:
        for f in self.files:
            try:
                f.mm.close()
            except BufferError:   # a view of the mapping is still alive somewhere: the mapping goes when it does
                pass
            f.fh.close()


def write_safetensors(path: str | Path, tensors: dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    """Writes one file; tensors in name order, data 8-byte aligned after the header."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in NAMES:
            raise WeightFileError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            fh.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
