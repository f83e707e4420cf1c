"""Loads the tensors a model declares from `model.safetensors` by name.

All declarations are checked against the file's header before anything is read; one error
lists every missing tensor, every tensor the model does not know and every wrong shape
(the reference stops at the first: src/lfm25_model.c:35-49, :296-317).

Types: in a bfloat16 run floating tensors stay bfloat16 (float16 is converted), a tensor stored
in 32-bit stays float32, integer tables become int32.  In a float32 run every floating tensor
becomes float32 (exact for bfloat16 and float16).
"""
from __future__ import annotations

import os
from typing import Iterable

import torch

from ..parts.base import WeightDecl
from .safetensors_io import SafetensorsError, SafetensorsFile

_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


class WeightsError(ValueError):
    """The checkpoint does not fit the model.  `.missing`, `.unexpected`, `.wrong_shape`
    (name, found, expected) and `.wrong_dtype` hold the details."""

    def __init__(self, path, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.path, self.missing, self.unexpected = path, list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = [f"{path} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, found, want in self.wrong_shape:
            lines.append(f"  tensor '{name}' has shape {list(found)}, expected {list(want)}")
        for name, found in self.wrong_dtype:
            lines.append(f"  tensor '{name}' has unsupported type {found}")
        super().__init__("\n".join(lines))


def _stored_name(decl: WeightDecl, names: set[str]):
    for n in (decl.name,) + tuple(decl.aliases):
        if n in names:
            return n
    return None


def check_header(path: str, st: SafetensorsFile, decls: Iterable[WeightDecl]) -> dict[str, str]:
    """Returns {declared name: stored name}; raises WeightsError listing everything wrong."""
    names = set(st.names())
    mapping, missing, wrong_shape, wrong_dtype = {}, [], [], []
    claimed = set()
    for d in decls:
        stored = _stored_name(d, names)
        if stored is None:
            missing.append(d.name)
            continue
        claimed.add(stored)
        mapping[d.name] = stored
        shape = st.shape(stored)
        if shape != tuple(d.shape) and shape not in tuple(tuple(s) for s in d.alt_shapes):
            wrong_shape.append((stored, shape, d.shape))
        if st.dtype(stored) not in _FLOATS + _INTS:
            wrong_dtype.append((stored, st.dtype(stored)))
    unexpected = sorted(names - claimed)
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(path, missing, unexpected, wrong_shape, wrong_dtype)
    return mapping


def target_dtype(stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if stored in _INTS:
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def load_weights(model_dir: str, decls: list[WeightDecl], run_dtype: torch.dtype,
                 device) -> dict[str, torch.Tensor]:
    path = os.path.join(model_dir, "model.safetensors")
    try:
        st = SafetensorsFile(path)
    except SafetensorsError as e:
        raise WeightsError(path, [], [], []) from e
    mapping = check_header(path, st, decls)
    out = {}
    for d in decls:
        t = st.read(mapping[d.name])
        t = t.reshape(d.shape).to(target_dtype(t.dtype, run_dtype))
        out[d.name] = t.to(device).contiguous()
    return out
