"""SwiGLU feed-forward: W_down (silu(W_gate h) * (W_up h)), silu(g) = g / (1 + exp(-g)).
Reference: src/lfm25_gpu.cu:583-618 (gate and up in one pass with the activation fused),
src/lfm25_engine.c:412-419.  Gate and up are one product; with bfloat16 weights their rows are
interleaved and the activation is the product's epilogue.
"""
from __future__ import annotations

from ..csrc import ops
from .base import FEED_FORWARDS, FeedForward, Runtime
from .linear import Linear


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, ffn_dim: int, *, names: dict[str, str],
                 aliases: dict[str, tuple] | None = None):
        """names: checkpoint names of 'gate' [F, d], 'up' [F, d], 'down' [d, F]."""
        self.d, self.F = int(hidden_size), int(ffn_dim)
        al = aliases or {}
        self.gate_up = Linear([names["gate"], names["up"]], self.d, [self.F, self.F],
                              aliases=[al.get("gate", ()), al.get("up", ())], swiglu_pair=True)
        self.down = Linear(names["down"], self.F, self.d, aliases=[al.get("down", ())])

    def weight_decls(self):
        return self.gate_up.weight_decls() + self.down.weight_decls()

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.gate_up.bind(weights, rt)
        self.down.bind(weights, rt)

    def forward(self, h, ctx, residual) -> None:
        if self.gate_up.interleaved:
            act = self.gate_up.forward(h, swiglu=True)          # silu(gate) * up in the product's epilogue
        else:
            gu = self.gate_up.forward(h)
            act = self.rt.empty(h.shape[0], self.F, dtype=gu.dtype)
            ops.swiglu(gu, act)
        self.down.forward(act, accumulate_into=residual)
