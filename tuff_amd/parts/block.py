"""Arrangements of parts around the residual stream.

PreNormBlock is the reference's layer (src/lfm25_engine.c:370-419):
    x += mixer(norm1(x));  x += ffn(norm2(x))
with the residual stream x in float32.  A feed-forward of None leaves out the second half.
"""
from __future__ import annotations

from typing import Optional

from .base import BLOCKS, Block, FeedForward, Mixer, Norm, Runtime


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Optional[Norm] = None,
                 ffn: Optional[FeedForward] = None):
        if (norm2 is None) != (ffn is None):
            raise ValueError("norm2 and ffn go together")
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn

    def _parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.ffn) if p is not None]

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._parts())

    def weight_decls(self):
        return [d for p in self._parts() for d in p.weight_decls()]

    def kernel_modules(self):
        return [m for p in self._parts() for m in p.kernel_modules()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)

    def forward(self, x, ctx, cache, write_cache: bool = True) -> None:
        h = self._normed(self.norm1, x, self.mixer)
        self.mixer.forward(h, ctx, cache, x, write_cache)
        if self.ffn is not None:
            h = self._normed(self.norm2, x, self.ffn)
            self.ffn.forward(h, ctx, x)

    @staticmethod
    def _normed(norm, x, consumer):
        """The norm of x for `consumer`: left pending if both sides know how (the consumer's first
        projection then runs the norm inside its kernel), else computed now."""
        if consumer.accepts_pending_norm and hasattr(norm, "pending"):
            return norm.pending(x)
        return norm.forward(x)
