"""Random-weights mode: from a configuration and a seed to tensors, or to a model folder
(config.json + model.safetensors) that loads like any other.

Matrices, embeddings and conv taps are N(0, 0.02); norm weights are 1 + N(0, 0.01).  Each
tensor has its own generator seeded by (seed, crc32 of its name), so a tensor's values do not
depend on which other tensors exist or in which order they are made.
"""
from __future__ import annotations

import json
import os
import zlib

import torch

from ..config.base import ModelConfig
from ..parts.base import WeightDecl
from .safetensors_io import write_safetensors

STD_MATRIX = 0.02
STD_NORM = 0.01


def random_tensor(decl: WeightDecl, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device)
    g.manual_seed((int(seed) * 0x9E3779B1 + zlib.crc32(decl.name.encode())) % (2 ** 63))
    t = torch.randn(tuple(decl.shape), generator=g, dtype=torch.float32, device=device)
    if decl.init == "norm":
        t = 1.0 + STD_NORM * t
    elif decl.init == "normal":
        t = STD_MATRIX * t
    else:
        raise ValueError(f"tensor '{decl.name}': unknown init '{decl.init}'")
    return t.to(dtype)


def random_weights(decls: list[WeightDecl], seed: int, run_dtype: torch.dtype, device,
                   stored_dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    """Tensors made on `device` directly: rounded to `stored_dtype` as a file would hold them,
    then kept in the type a run of `run_dtype` keeps them in."""
    from .loader import target_dtype
    out = {}
    for d in decls:
        t = random_tensor(d, seed, stored_dtype, device)
        out[d.name] = t.to(target_dtype(stored_dtype, run_dtype)).contiguous()
    return out


def write_random_model(cfg: ModelConfig, out_dir: str, seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Writes config.json and model.safetensors for `cfg` into out_dir and returns out_dir."""
    from ..models.registry import build_model
    model = build_model(cfg)
    decls = {d.name: d for d in model.weight_decls()}
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f, indent=2)
    write_safetensors(
        os.path.join(out_dir, "model.safetensors"),
        [(d.name, tuple(d.shape), dtype) for d in decls.values()],
        lambda name: random_tensor(decls[name], seed, dtype),
        metadata={"format": "pt", "seed": seed})
    return out_dir
