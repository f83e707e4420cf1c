"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, in float32 (src/lfm25_gpu.cu:235,244)."""
from __future__ import annotations

from typing import Optional

import torch

from ..csrc import ops
from .base import NORMS, Norm, Runtime, WeightDecl


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, dim: int, eps: float, name: str, aliases: tuple = ()):
        self.dim, self.eps, self.name, self.aliases = int(dim), float(eps), name, tuple(aliases)
        self.weight: Optional[torch.Tensor] = None

    def weight_decls(self):
        return [WeightDecl(self.name, (self.dim,), "norm", aliases=self.aliases)]

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.weight = weights[self.name]

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = self.rt.empty(n, self.dim)
        ops.rmsnorm(x, self.weight, out, self.eps, rows)
        return out
