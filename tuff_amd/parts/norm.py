"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, in float32 (src/lfm25_gpu.cu:235,244)."""
from __future__ import annotations

from typing import Optional

import torch

from ..csrc import ops
from .base import NORMS, Norm, Runtime, WeightDecl


class PendingNorm:
    """An RMSNorm that has not run yet: the float32 rows, the weight and eps.  A projection that
    can apply the norm inside its own kernel takes it as it is; anything else calls tensor(),
    which runs the norm kernel once."""

    def __init__(self, norm: "RMSNorm", x: torch.Tensor, rows: Optional[torch.Tensor], pre=None):
        self.norm, self.x, self.rows = norm, x, rows
        self.pre = pre            # (xw, ss) left by the product that last added into x, or None
        self._tensor: Optional[torch.Tensor] = None

    @property
    def shape(self):
        n = self.x.shape[0] if self.rows is None else self.rows.shape[0]
        return (n, self.norm.dim)

    @property
    def dtype(self):
        return self.norm.rt.dtype

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.x, self.rows)
        return self._tensor


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    records_portions = True

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
        self.weight_f32 = self.weight if self.weight.dtype == torch.float32 else self.weight.float()

    def pending(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> PendingNorm:
        """The norm of x as a PendingNorm, for consumers that say they accept one."""
        pre = self.take_announced(x)
        return PendingNorm(self, x, rows, pre if rows is None else None)

    def take_announced(self, x: torch.Tensor):
        """(xw, ss) if the product that last added into x announced them, else None; either way nothing stays."""
        ready, self._ready = getattr(self, "_ready", None), None
        return ready[1:] if ready is not None and ready[0] is x else None

    def announce_operand(self, x: torch.Tensor, xw: torch.Tensor, ss: torch.Tensor) -> None:
        """Called by the product that has just added into x and, in the same kernel, written
        xw = bf16(x * weight) and the per-tile sums of squares ss: the next pending(x) carries them."""
        self._ready = (x, xw, ss)

    def forget(self) -> None:
        """Drops what announce_operand() left, if nobody asked for it (end of a step)."""
        self._ready = None

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = self.rt.empty(n, self.dim)
        ops.rmsnorm(x, self.weight, out, self.eps, rows)
        return out
