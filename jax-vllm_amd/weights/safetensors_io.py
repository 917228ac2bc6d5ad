"""Minimal reader and writer of the safetensors container, by tensor name.

Format: 8 bytes little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}``, then
the tensors' bytes.  The reader memory-maps the file and hands out zero-copy CPU views,
so a large checkpoint is streamed to the GPU tensor by tensor and never held whole.
"""
from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path
from typing import Iterable, Iterator

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFormatError(ValueError):
    pass


class SafetensorsFile:
    """One ``.safetensors`` file, memory-mapped.  ``entries`` maps name -> (dtype, shape)."""

    def __init__(self, path):
        self.path = Path(path)
        self._f = open(self.path, "rb")
        head = self._f.read(8)
        if len(head) != 8:
            raise SafetensorsFormatError(f"{self.path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = self.path.stat().st_size
        if n > size - 8:
            raise SafetensorsFormatError(f"{self.path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._f.read(n))
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise SafetensorsFormatError(f"{self.path}: header is not JSON: {e}") from e
        self._base = 8 + n
        self.metadata = header.pop("__metadata__", {})
        self._raw = header
        self.entries = {}
        for name, e in header.items():
            if e["dtype"] not in _DTYPES:
                raise SafetensorsFormatError(f"{self.path}: tensor {name!r} has unsupported dtype {e['dtype']}")
            b, end = e["data_offsets"]
            dtype, shape = _DTYPES[e["dtype"]], tuple(e["shape"])
            count = 1
            for s in shape:
                count *= s
            if end - b != count * dtype.itemsize or self._base + end > size:
                raise SafetensorsFormatError(f"{self.path}: tensor {name!r} has inconsistent offsets")
            self.entries[name] = (dtype, shape)
        # a private copy-on-write map: torch wants a writable buffer, nothing is ever written
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_COPY) if size > 0 else None

    def tensor(self, name: str) -> torch.Tensor:
        """Zero-copy CPU view of one tensor (valid while this object lives)."""
        dtype, shape = self.entries[name]
        b, end = self._raw[name]["data_offsets"]
        if end == b:
            return torch.empty(shape, dtype=dtype)
        flat = torch.frombuffer(self._mm, dtype=dtype, count=(end - b) // dtype.itemsize, offset=self._base + b)
        return flat.view(shape)

    def close(self) -> None:
        # views handed out keep the map alive through their buffer reference
        self._f.close()


def write_safetensors(path, tensors: Iterable, metadata: dict | None = None) -> None:
    """Write ``(name, shape, dtype, make)`` records, where ``make()`` returns the CPU tensor;
    tensors are produced and written one at a time."""
    records = list(tensors)
    header, offset = {}, 0
    for name, shape, dtype, _ in records:
        count = 1
        for s in shape:
            count *= s
        nbytes = count * dtype.itemsize
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype, make in records:
            t = make().contiguous()
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise ValueError(f"tensor {name!r} was produced as {tuple(t.shape)} {t.dtype}, declared {shape} {dtype}")
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")


def open_shards(folder) -> Iterator[SafetensorsFile]:
    """Every ``*.safetensors`` of a folder in sorted order (reference: ``jllm/model/weights.py:21-30``)."""
    shards = sorted(Path(folder).glob("*.safetensors"))
    if not shards:
        raise FileNotFoundError(f"no safetensors in {folder}")
    for s in shards:
        yield SafetensorsFile(s)
