"""The safetensors container, read and written without a library: an 8-byte
little-endian header length, a JSON header {name: {dtype, shape, data_offsets}},
then the raw little-endian data.  Takes the place of the reference's GGUF reader
(src/gguf/mod.rs:166-255: header, tensor table, `tensor_view(name)`)."""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A memory-mapped file; `tensor(name)` is a view into the map (no copy)."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"cannot open {path}: {e.strerror}") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._f.read(n))
        except ValueError as e:
            raise SafetensorsError(f"{path}: header is no JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {})
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_COPY)
        self._base = 8 + n
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            if e["dtype"] not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unknown dtype {e['dtype']}")
            dtype = _DTYPES[e["dtype"]]
            shape = tuple(int(s) for s in e["shape"])
            lo, hi = e["data_offsets"]
            count = 1
            for s in shape:
                count *= s
            if hi - lo != count * dtype.itemsize or self._base + hi > size:
                raise SafetensorsError(f"{path}: tensor {name} has offsets {lo}..{hi} that do not fit shape {list(shape)} {e['dtype']}")
            self.entries[name] = (dtype, shape, lo, hi)

    def names(self) -> List[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, lo, hi = self.entries[name]
        if hi == lo:
            return torch.empty(shape, dtype=dtype)
        count = (hi - lo) // dtype.itemsize
        flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._base + lo)
        return flat.view(shape)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] | None = None) -> None:
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = metadata
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.dtype.itemsize
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
