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

    @property
    def records_portions(self):
        return all(p.records_portions for p in self._parts())

    def weight_decls(self):
        return [d for p in self._parts() for d in p.weight_decls()]

    def kernel_modules(self):
        return [m for p in self._parts() for m in p.kernel_modules()]

    def token_inputs(self):
        return [t for p in self._parts() for t in p.token_inputs()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)

    takes_next_norm = True

    def first_norm_consumer(self):
        """(norm, part that consumes it) at the head of the block, for the block before this one."""
        return self.norm1, self.mixer

    def forward(self, x, ctx, cache, write_cache: bool = True, next_norm=None) -> None:
        """next_norm: (norm, consumer) that will read x right after this block, or None."""
        h = self._normed(self.norm1, x, self.mixer)
        after = self._hand_over(self.mixer, (self.norm2, self.ffn) if self.ffn is not None else next_norm)
        self.mixer.forward(h, ctx, cache, x, write_cache, **after)
        if self.ffn is not None:
            h = self._normed(self.norm2, x, self.ffn)
            after = self._hand_over(self.ffn, next_norm)
            self.ffn.forward(h, ctx, x, **after)

    def forget(self) -> None:
        """End of a step: drops what a product left for a norm that never asked for it."""
        for n in (self.norm1, self.norm2):
            if hasattr(n, "forget"):
                n.forget()

    @staticmethod
    def _hand_over(producer, nxt) -> dict:
        """The keyword that tells the producer's last projection which norm reads x next: only if
        producer, norm and the norm's consumer all know how (else nothing is passed and the norm
        runs as a kernel of its own)."""
        if not producer.adds_once_through_linear:
            return {}
        ok = (nxt is not None and hasattr(nxt[0], "announce_operand") and nxt[1] is not None
              and nxt[1].accepts_pending_norm)
        return {"next_norm": nxt[0] if ok else None}

    @staticmethod
    def _normed(norm, x, consumer):
        """The norm of x for `consumer`: left pending if both sides know how (the consumer's first
        projection then runs the norm inside its kernel), else computed now."""
        if consumer.accepts_pending_norm and hasattr(norm, "pending"):
            return norm.pending(x)
        return norm.forward(x)
