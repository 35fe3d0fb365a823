"""Reading and writing safetensors files: an 8-byte little-endian header length,
a JSON header `{name: {dtype, shape, data_offsets}}`, then the raw tensor bytes.

Tensors are read by name through a memory map, so a large file is never loaded
whole; nothing in a file is executed.
"""

from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path
from typing import Iterable, Iterator

import numpy as np
import torch

_DTYPES: dict[str, torch.dtype] = {
    "F64": torch.float64,
    "F32": torch.float32,
    "F16": torch.float16,
    "BF16": torch.bfloat16,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: tuple[int, ...]
    begin: int
    end: int
    file: Path

    @property
    def is_integer(self) -> bool:
        return not self.dtype.is_floating_point

    @property
    def is_32bit_float(self) -> bool:
        return self.dtype == torch.float32


class SafetensorsFile:
    """One file, opened lazily; `entries` after construction, tensors on demand."""

    def __init__(self, path: str | Path) -> None:
        self.path = Path(path)
        with open(self.path, "rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise SafetensorsError(f"{self.path}: too short for a safetensors file")
            (length,) = struct.unpack("<Q", head)
            size = self.path.stat().st_size
            if length <= 0 or 8 + length > size:
                raise SafetensorsError(f"{self.path}: header length {length} does not fit the file")
            try:
                header = json.loads(f.read(length).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as e:
                raise SafetensorsError(f"{self.path}: header is not JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{self.path}: header must be a JSON object")
        self.data_start = 8 + length
        self.metadata = header.pop("__metadata__", None)
        self.entries: dict[str, TensorEntry] = {}
        for name, info in header.items():
            try:
                dtype = _DTYPES[info["dtype"]]
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError) as e:
                raise SafetensorsError(f"{self.path}: bad header entry for {name!r}: {e}") from None
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if end - begin != count * dtype.itemsize or begin < 0 or self.data_start + end > size:
                raise SafetensorsError(f"{self.path}: data range of {name!r} does not fit its shape or the file")
            self.entries[name] = TensorEntry(name, dtype, shape, begin, end, self.path)
        self._map: mmap.mmap | None = None
        self._fh = None

    def _buffer(self) -> mmap.mmap:
        if self._map is None:
            self._fh = open(self.path, "rb")
            self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        return self._map

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor copied out of the map (the map can be closed afterwards)."""
        e = self.entries[name]
        count = int(np.prod(e.shape, dtype=np.int64)) if e.shape else 1
        if count == 0:
            return torch.empty(e.shape, dtype=e.dtype)
        raw = np.frombuffer(self._buffer(), dtype=np.uint8, count=e.end - e.begin, offset=self.data_start + e.begin)
        return torch.from_numpy(raw.copy()).view(e.dtype).reshape(e.shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        if self._fh is not None:
            self._fh.close()
            self._fh = None

    def __enter__(self) -> "SafetensorsFile":
        return self

    def __exit__(self, *exc) -> None:
        self.close()


def write_safetensors(
    path: str | Path,
    layout: Iterable[tuple[str, torch.dtype, tuple[int, ...]]],
    tensors: Iterator[tuple[str, torch.Tensor]],
    metadata: dict[str, str] | None = None,
) -> None:
    """Write a file whose header is known up front (`layout`) while `tensors`
    streams the data in the same order, one tensor in memory at a time."""
    header: dict[str, object] = {}
    if metadata:
        header["__metadata__"] = metadata
    offset = 0
    order: list[tuple[str, torch.dtype, tuple[int, ...]]] = []
    for name, dtype, shape in layout:
        if name in header:
            raise SafetensorsError(f"tensor {name!r} listed twice")
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        size = count * dtype.itemsize
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + size]}
        offset += size
        order.append((name, dtype, tuple(shape)))
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for (name, dtype, shape), (got_name, tensor) in zip(order, tensors, strict=True):
            if got_name != name or tensor.dtype != dtype or tuple(tensor.shape) != shape:
                raise SafetensorsError(
                    f"stream gave {got_name!r} {tensor.dtype} {tuple(tensor.shape)}, "
                    f"the header expects {name!r} {dtype} {shape}"
                )
            data = tensor.detach().cpu().contiguous()
            f.write(data.view(torch.uint8).numpy().tobytes() if data.numel() else b"")


def save_state_dict(path: str | Path, tensors: dict[str, torch.Tensor]) -> None:
    """Convenience for small models and tests."""
    layout = [(n, t.dtype, tuple(t.shape)) for n, t in tensors.items()]
    write_safetensors(path, layout, iter(tensors.items()))
