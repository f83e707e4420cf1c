"""Rotary position encoding.  theta_j = base^(-2j / rotary_dim); the pair of channels that
shares theta_j is (j, j + rotary_dim/2) in the half-split form the reference uses
(src/lfm25_gpu.cu:459-474) or (2j, 2j + 1) in the interleaved form.  theta is computed in
float64 once and rounded to float32; angle, cosine and sine are float32 in the kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import POSITION_ENCODINGS, PositionEncoding, Runtime


_TABLES: dict = {}          # (device, base, rotary_dim, positions) -> table, shared between layers


@POSITION_ENCODINGS.register("rotary")
class Rotary(PositionEncoding):
    graph_safe = True
    records_portions = True

    def __init__(self, head_dim: int, base: float, rotary_dim: Optional[int] = None,
                 interleaved: bool = False, table_positions: Optional[int] = None):
        """table_positions: keep the cosines and sines of this many positions in a table on the device
        (shared by all encodings of the same base and size) for kernels that would otherwise spend
        more time on computing them than on the rest of their work."""
        self.head_dim, self.base = int(head_dim), float(base)
        self.table_positions = int(table_positions) if table_positions else 0
        self.angles: Optional[torch.Tensor] = None
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        self.interleaved = bool(interleaved)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within the head size "
                             f"{self.head_dim}")
        self.inv_freq: Optional[torch.Tensor] = None

    def kernel_modules(self):
        return ["rope_kv"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        j = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        inv = torch.tensor(self.base, dtype=torch.float64) ** (-2.0 * j / self.rotary_dim)
        self.inv_freq = inv.to(torch.float32).to(rt.device)
        if self.table_positions and rt.device.type == "cuda":
            from ..csrc import ops
            key = (str(rt.device), self.base, self.rotary_dim, self.table_positions)
            if key not in _TABLES:
                while len(_TABLES) >= 4:             # tables of models long gone
                    _TABLES.pop(next(iter(_TABLES)))
                _TABLES[key] = ops.rope_table(self.inv_freq, self.table_positions)
            self.angles = _TABLES[key]

    def angle_table(self) -> Optional[torch.Tensor]:
        """float32 [positions, 2, rotary_dim / 2] (cosines, sines) or None."""
        return self.angles

    def rotary_tables(self):
        return self.inv_freq, self.rotary_dim, self.interleaved
