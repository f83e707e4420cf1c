"""Reading and writing the safetensors container: 8 bytes little-endian header length, a JSON
header {name: {dtype, shape, data_offsets}}, then the raw tensors.  Tensors are read one at a
time by name, so a model never has to fit in host memory twice.
"""
from __future__ import annotations

import json
import os
import struct
from typing import Iterable, Iterator

import torch

_DTYPES = {
    "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """Header of one .safetensors file and by-name access to its tensors."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise SafetensorsError(f"no such file: {path}")
        size = os.path.getsize(path)
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise SafetensorsError(f"{path}: too short to be a safetensors file")
            (n,) = struct.unpack("<Q", head)
            if n <= 0 or 8 + n > size:
                raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
            try:
                header = json.loads(f.read(n))
            except (json.JSONDecodeError, UnicodeDecodeError) as e:
                raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        self.data_start = 8 + n
        self.metadata = header.pop("__metadata__", {}) or {}
        self.entries: dict[str, dict] = {}
        for name, e in header.items():
            try:
                dt, shape, (b, en) = e["dtype"], tuple(int(s) for s in e["shape"]), e["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed entry for tensor '{name}'") from None
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            numel = 1
            for s in shape:
                numel *= s
            nbytes = numel * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if en - b != nbytes or b < 0 or self.data_start + en > size:
                raise SafetensorsError(f"{path}: tensor '{name}' data range [{b}, {en}) does not match "
                                       f"shape {list(shape)} of {dt}")
            self.entries[name] = {"dtype": _DTYPES[dt], "shape": shape, "begin": b, "end": en}

    def names(self) -> list[str]:
        return list(self.entries)

    def shape(self, name: str) -> tuple:
        return self.entries[name]["shape"]

    def dtype(self, name: str) -> torch.dtype:
        return self.entries[name]["dtype"]

    def read(self, name: str) -> torch.Tensor:
        e = self.entries[name]
        with open(self.path, "rb") as f:
            f.seek(self.data_start + e["begin"])
            buf = bytearray(e["end"] - e["begin"])
            got = f.readinto(buf)
        if got != len(buf):
            raise SafetensorsError(f"{self.path}: short read of tensor '{name}'")
        if len(buf) == 0:
            return torch.empty(e["shape"], dtype=e["dtype"])
        return torch.frombuffer(buf, dtype=e["dtype"]).reshape(e["shape"])


def write_safetensors(path: str, tensors: Iterable[tuple[str, tuple, torch.dtype]],
                      produce, metadata: dict | None = None) -> None:
    """Writes tensors one after the other.  `tensors` lists (name, shape, dtype) in file order;
    `produce(name)` returns the CPU tensor when its turn comes."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    plan = []
    for name, shape, dtype in tensors:
        if dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {dtype}")
        numel = 1
        for s in shape:
            numel *= int(s)
        nbytes = numel * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAMES[dtype], "shape": [int(s) for s in shape],
                        "data_offsets": [offset, offset + nbytes]}
        plan.append((name, tuple(int(s) for s in shape), dtype, nbytes))
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype, nbytes in plan:
            t = produce(name)
            if tuple(t.shape) != shape or t.dtype != dtype:
                raise SafetensorsError(f"tensor '{name}': produced {tuple(t.shape)} {t.dtype}, "
                                       f"declared {shape} {dtype}")
            raw = t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes() if nbytes else b""
            f.write(raw)
    os.replace(tmp, path)
