"""SwiGLU feed-forward: W_down (silu(W_gate h) * (W_up h)), silu(g) = g / (1 + exp(-g)).
Reference: src/lfm25_gpu.cu:583-618 (gate and up in one pass with the activation fused),
src/lfm25_engine.c:412-419.  Gate and up are one product; with bfloat16 weights their rows are
interleaved and the activation is the product's epilogue.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import FEED_FORWARDS, FeedForward, Runtime
from .linear import Linear


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    records_portions = True
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, ffn_dim: int, *, names: dict[str, str],
                 aliases: dict[str, tuple] | None = None):
        """names: checkpoint names of 'gate' [F, d], 'up' [F, d], 'down' [d, F]."""
        self.d, self.F = int(hidden_size), int(ffn_dim)
        self._names, self._al = dict(names), aliases or {}
        self._make(self.F)
        self._decls = self.gate_up.weight_decls() + self.down.weight_decls()

    def _make(self, width: int) -> None:
        names, al = self._names, self._al
        self.gate_up = Linear([names["gate"], names["up"]], self.d, [width, width],
                              aliases=[al.get("gate", ()), al.get("up", ())], swiglu_pair=True)
        self.down = Linear(names["down"], width, self.d, aliases=[al.get("down", ())])
        self.width = width

    def weight_decls(self):
        return self._decls

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        names = self._names
        g, u, dn = (weights[names[k]] for k in ("gate", "up", "down"))
        if self.F % 8 and all(t.dtype == torch.bfloat16 for t in (g, u, dn)):
            # The bfloat16 matrix kernels read 16 bytes at a time along the inner size.  A width that is
            # no multiple of 8 is filled up with zero rows of gate and up (silu(0) * 0 = 0, exactly) and
            # zero columns of down: the same function.
            pad = -self.F % 8
            weights = dict(weights)
            weights[names["gate"]] = torch.cat([g, g.new_zeros(pad, self.d)])
            weights[names["up"]] = torch.cat([u, u.new_zeros(pad, self.d)])
            weights[names["down"]] = torch.cat([dn, dn.new_zeros(self.d, pad)], dim=1).contiguous()
            self._make(self.F + pad)
        self.gate_up.bind(weights, rt)
        self.down.bind(weights, rt)

    def forward(self, h, ctx, residual, next_norm=None) -> None:
        if self.gate_up.interleaved:
            act = self.gate_up.forward(h, swiglu=True)          # silu(gate) * up in the product's epilogue
        else:
            gu = self.gate_up.forward(h)
            act = self.rt.empty(h.shape[0], self.width, dtype=gu.dtype)
            ops.swiglu(gu, act)
        self.down.forward(act, accumulate_into=residual, next_norm=next_norm)
