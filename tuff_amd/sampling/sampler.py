"""Draws the next token of every request of a step from its logits row, on the GPU.

Per request: greedy if temp <= 0 (the penalty is not applied then, as in the reference's
fast path, src/sampler.c:102-113); else repetition penalty -> min-p -> top-k -> top-p -> draw
with the request's own xorshift128+ generator.  The uniform is drawn on the host, one per
stochastic row, so a request's stream does not depend on what else is in the batch.

Not the reference's arithmetic at the borders of the cumulative sums: the reference adds its float32
probabilities one after the other (src/sampler.c:185-226), so its running sum carries up to one rounding a
term and the candidate at which it reaches top_p, or the draw, is uncertain by that much probability (at a
vocabulary of 47,000 to 65,000: candidates 20 to 100 places apart, all of them of tiny probability).  The kernel
adds 40-bit fixed-point probabilities exactly, whatever the order, and picks what float64 sums pick.  The same
seed and logits can therefore give another token than the reference's sampler where the draw falls that close to
a border; with small vocabularies or sharp distributions they agree.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from ..csrc import ops
from .params import SamplerState


class PendingSample:
    """Tokens that are being drawn: `out` (int32 [R], device) is valid for kernels launched after
    this one on the same stream; tokens() waits for the copy to the host."""

    def __init__(self, out: torch.Tensor, states: Sequence[SamplerState]):
        self.out, self.states = out, list(states)
        self.host = torch.empty(out.shape, dtype=torch.int32, pin_memory=True)
        self.host.copy_(out, non_blocking=True)
        self.done = torch.cuda.Event()
        self.done.record()
        self._tokens = None

    def tokens(self) -> list[int]:
        if self._tokens is None:
            self.done.synchronize()
            self._tokens = self.host.tolist()
            for s, t in zip(self.states, self._tokens):
                s.accept(t)
        return self._tokens


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample(self, logits: torch.Tensor, states: Sequence[SamplerState]) -> list[int]:
        """logits: float32 [R, vocab] on the device (changed in place where a penalty applies);
        states: the R requests' sampler states, in row order.  Returns R token ids and records
        them in the states' rings."""
        if logits.shape[0] == 0 and not states:
            return []
        return self.launch(logits, states).tokens()

    @staticmethod
    def needs_history(state: SamplerState) -> bool:
        """The draw depends on the request's earlier tokens (repetition penalty)."""
        return state.params.temp > 0.0 and state.params.repeat_penalty > 1.0

    def _upload(self, array: np.ndarray) -> torch.Tensor:
        """To the device through pinned memory, without making the host wait for the stream."""
        return torch.from_numpy(array).pin_memory().to(self.device, non_blocking=True)

    def launch(self, logits: torch.Tensor, states: Sequence[SamplerState]) -> PendingSample:
        """Starts the draw and returns without waiting for it."""
        R = logits.shape[0]
        if R != len(states):
            raise ValueError(f"{R} logits rows for {len(states)} requests")
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        stochastic = [s.params.temp > 0.0 for s in states]
        if not any(stochastic):
            ops.sample(logits, out)
        else:
            f32 = np.zeros((5, R), dtype=np.float32)      # temp, top_p, min_p, uniform, penalty
            top_k = np.zeros(R, dtype=np.int32)
            for r, s in enumerate(states):
                p = s.params
                f32[0, r], f32[1, r], f32[2, r], f32[4, r] = p.temp, p.top_p, p.min_p, 1.0
                top_k[r] = p.top_k
                if stochastic[r]:
                    f32[3, r] = s.rng.uniform()
                    f32[4, r] = p.repeat_penalty
            dev = self._upload(f32)
            penalised = [r for r, s in enumerate(states)
                         if stochastic[r] and s.params.repeat_penalty > 1.0 and s.count > 0]
            if penalised:
                cap = max(states[r].cap for r in penalised)
                recent = np.zeros((R, cap), dtype=np.int32)
                counts = np.zeros(R, dtype=np.int32)
                for r in penalised:
                    recent[r, :states[r].count] = states[r].recent[:states[r].count]
                    counts[r] = states[r].count
                ops.repeat_penalty(logits, self._upload(recent), self._upload(counts), dev[4].contiguous())
            ops.sample(logits, out, temps=dev[0].contiguous(), top_ks=self._upload(top_k),
                       top_ps=dev[1].contiguous(), min_ps=dev[2].contiguous(), uniforms=dev[3].contiguous())
        return PendingSample(out, states)
