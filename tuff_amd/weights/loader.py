"""Loads the tensors a model declares from `model.safetensors` by name (or from the files that a
`model.safetensors.index.json` names: {"weight_map": {tensor name: file name}}).

All declarations are checked against the headers before anything is read; one error lists every
missing tensor, every tensor the model does not know and every wrong shape (the reference stops
at the first: src/lfm25_model.c:35-49, :296-317).  Tensors the model does not know are, alone, no
error: a required tensor must be there, others may (src/lfm25_model.c:35-49 binds by name and
never looks at the rest of the file); they are listed once in an UnexpectedTensorsWarning, or in
the error under strict=True.

Types: in a bfloat16 run floating tensors stay bfloat16 (float16 is converted), a tensor stored
in 32-bit stays float32, integer tables become int32.  In a float32 run every floating tensor
becomes float32 (exact for bfloat16 and float16).
"""
from __future__ import annotations

import json
import os
import warnings
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


class UnexpectedTensorsWarning(UserWarning):
    """The checkpoint holds tensors that the model does not declare; `.names` lists them."""

    def __init__(self, path, names):
        self.path, self.names = path, list(names)
        super().__init__(f"{path}: {len(self.names)} tensors that the model does not know are ignored: "
                         + ", ".join(self.names))


class Checkpoint:
    """The tensors of one model folder by name, whichever file holds them."""

    def __init__(self, model_dir: str):
        single = os.path.join(model_dir, "model.safetensors")
        index = single + ".index.json"
        self.path = single
        self.where: dict[str, SafetensorsFile] = {}
        if os.path.isfile(single) or not os.path.isfile(index):
            st = SafetensorsFile(single)
            self.where = {n: st for n in st.names()}
            return
        self.path = index
        try:
            with open(index) as f:
                weight_map = json.load(f)["weight_map"]
            if not isinstance(weight_map, dict):
                raise TypeError("weight_map is no object")
        except (OSError, ValueError, KeyError, TypeError) as e:
            raise SafetensorsError(f"{index}: not an index of safetensors files ({e})") from None
        files: dict[str, SafetensorsFile] = {}
        for name, fn in weight_map.items():
            if fn not in files:
                if os.path.basename(str(fn)) != fn:
                    raise SafetensorsError(f"{index}: file name '{fn}' leaves the model folder")
                files[fn] = SafetensorsFile(os.path.join(model_dir, fn))
            if name not in files[fn].entries:
                raise SafetensorsError(f"{index}: tensor '{name}' is not in {fn}")
            self.where[name] = files[fn]

    def names(self) -> list[str]:
        return list(self.where)

    def shape(self, name: str) -> tuple:
        return self.where[name].shape(name)

    def dtype(self, name: str) -> torch.dtype:
        return self.where[name].dtype(name)

    def read(self, name: str) -> torch.Tensor:
        return self.where[name].read(name)


def _stored_name(decl: WeightDecl, names: set[str]):
    for n in (decl.name,) + tuple(decl.aliases):
        if n in names:
            return n
    return None


def check_header(path: str, st, decls: Iterable[WeightDecl], strict: bool = False) -> dict[str, str]:
    """Returns {declared name: stored name}; raises WeightsError listing everything wrong.  Tensors that
    no declaration claims: part of that error's list; alone, a warning (an error under `strict`)."""
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
    if missing or wrong_shape or wrong_dtype or (unexpected and strict):
        raise WeightsError(path, missing, unexpected, wrong_shape, wrong_dtype)
    if unexpected:
        warnings.warn(UnexpectedTensorsWarning(path, unexpected), stacklevel=3)
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
                 device, strict: bool = False) -> dict[str, torch.Tensor]:
    try:
        st = Checkpoint(model_dir)
    except SafetensorsError as e:
        raise WeightsError(os.path.join(model_dir, "model.safetensors"), [], [], []) from e
    mapping = check_header(st.path, st, decls, strict)
    out = {}
    for d in decls:
        t = st.read(mapping[d.name])
        t = t.reshape(d.shape).to(target_dtype(t.dtype, run_dtype))
        out[d.name] = t.to(device).contiguous()
    return out
