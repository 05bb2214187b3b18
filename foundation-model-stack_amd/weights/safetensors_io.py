"""Reading and writing the safetensors file layout without loading a file whole.

Layout: 8 bytes little-endian header length, a JSON header mapping each tensor
name to dtype, shape and byte offsets, then the raw little-endian data.
Tensors are read one by one from a memory map (the reference reads lazily for
the same reason, fms/utils/serialization.py:319-336), and written one by one,
so a model larger than host memory can pass through.
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Iterator, List, Tuple

import torch

_DTYPES = {
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


class SafetensorsFile:
    """The tensors of one file, by name, read on demand."""

    def __init__(self, path: str):
        self.path = path
        self._file = open(path, "rb")
        head = self._file.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: not a safetensors file (shorter than its header length)")
        (n,) = struct.unpack("<Q", head)
        size = os.path.getsize(path)
        if n > size - 8:
            raise ValueError(f"{path}: header length {n} exceeds the file")
        header = json.loads(self._file.read(n))
        self._data_start = 8 + n
        self.entries: Dict[str, dict] = {k: v for k, v in header.items() if k != "__metadata__"}
        for name, meta in self.entries.items():
            lo, hi = meta["data_offsets"]
            if meta["dtype"] not in _DTYPES or lo > hi or self._data_start + hi > size:
                raise ValueError(f"{path}: tensor {name!r} has a bad header entry")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def keys(self) -> List[str]:
        return list(self.entries)

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]]

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.entries[name]["shape"])

    def read(self, name: str) -> torch.Tensor:
        meta = self.entries[name]
        lo, hi = meta["data_offsets"]
        dtype = _DTYPES[meta["dtype"]]
        if hi == lo:
            return torch.empty(meta["shape"], dtype=dtype)
        buf = memoryview(self._map)[self._data_start + lo : self._data_start + hi]
        # a private copy: the map goes away with the file
        return torch.frombuffer(bytearray(buf), dtype=dtype).reshape(meta["shape"])

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        self._file.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, Tuple[int, ...], torch.dtype]], produce) -> None:
    """Write a file from (name, shape, dtype) entries; `produce(name)` returns each tensor when its turn comes."""
    entries = list(tensors)
    header = {}
    offset = 0
    for name, shape, dtype in entries:
        count = 1
        for s in shape:
            count *= s
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype in entries:
            t = produce(name)
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise ValueError(f"{name}: produced {tuple(t.shape)} {t.dtype}, declared {tuple(shape)} {dtype}")
            t = t.contiguous()
            if t.dtype == torch.bfloat16:
                f.write(t.view(torch.int16).numpy().tobytes())
            else:
                f.write(t.numpy().tobytes())
    os.replace(tmp, path)


def iter_tensors(file: SafetensorsFile) -> Iterator[Tuple[str, torch.Tensor]]:
    for name in file.keys():
        yield name, file.read(name)
