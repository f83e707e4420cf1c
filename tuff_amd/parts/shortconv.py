"""Gated short-convolution mixer with per-request state.

bcx = W_in h; B, C, X = thirds of bcx; u = B * X; y_t = sum_k w[:, k] u_{t-(K-1)+k}; the
request's state keeps the last K-1 rows of u; o = W_out (C * y).
Reference: src/lfm25_gpu.cu:378-397 and :1056-1079, src/lfm25_engine.c:376-380; no biases
(src/lfm25_model.c:154-163).
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import MIXERS, FixedState, Mixer, Runtime, WeightDecl
from .linear import Linear

MAX_KERNEL = 17      # the state kernel keeps K-1 <= 16 rows in registers


@MIXERS.register("shortconv")
class ShortConvMixer(Mixer):
    graph_safe = True
    records_portions = True
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, kernel_size: int, *, names: dict[str, str],
                 aliases: dict[str, tuple] | None = None):
        """names: checkpoint names of 'in_proj' [3d, d], 'conv' [d, K], 'out_proj' [d, d]."""
        self.d, self.K = int(hidden_size), int(kernel_size)
        if not 2 <= self.K <= MAX_KERNEL:
            raise ValueError(f"short-conv kernel size {self.K} is outside the supported 2..{MAX_KERNEL}")
        al = aliases or {}
        self.names = dict(names)
        self.in_proj = Linear(names["in_proj"], self.d, 3 * self.d, aliases=[al.get("in_proj", ())])
        self.out_proj = Linear(names["out_proj"], self.d, self.d, aliases=[al.get("out_proj", ())])
        self._al = al
        self.conv_w = None

    def weight_decls(self):
        return (self.in_proj.weight_decls() + self.out_proj.weight_decls() +
                [WeightDecl(self.names["conv"], (self.d, self.K), "normal",
                            alt_shapes=((self.d, 1, self.K),), aliases=self._al.get("conv", ()))])

    def kernel_modules(self):
        return ["shortconv"]

    def cache_spec(self):
        return FixedState((self.K - 1, self.d))

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.in_proj.bind(weights, rt)
        self.out_proj.bind(weights, rt)
        self.conv_w = weights[self.names["conv"]].reshape(self.d, self.K).contiguous()
        # bfloat16: projection and convolution of single tokens in one kernel, from a regrouped copy of the weight
        self.in_proj.group_rows_for_conv()

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        T = h.shape[0]
        if write_cache and ctx.max_q_len == 1:
            y = self.in_proj.forward_conv(h, conv_w=self.conv_w, state=cache.state, state_slot=ctx.state_slot)
            if y is not None:
                self.out_proj.forward(y, accumulate_into=residual, next_norm=next_norm)
                return
        bcx = self.in_proj.forward(h)
        y = self.rt.empty(T, self.d)
        if write_cache and ctx.max_q_len == 1:
            # single tokens only: one kernel reads the state, writes the output and the new state
            ops.shortconv_decode(bcx, self.conv_w, cache.state, y, state_slot=ctx.state_slot, K=self.K)
            self.out_proj.forward(y, accumulate_into=residual, next_norm=next_norm)
            return
        # output and, unless the cache is only read, the new state in one kernel
        ops.shortconv_fwd(bcx, self.conv_w, cache.state, y, req_of_token=ctx.req_of_token,
                          q_start=ctx.q_start, state_slot=ctx.state_slot, K=self.K,
                          q_len=ctx.q_len if write_cache else None)
        self.out_proj.forward(y, accumulate_into=residual, next_norm=next_norm)
