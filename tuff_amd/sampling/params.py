"""Sampling options, with the names, defaults and meanings of the reference
(include/sampler.h:12-20, src/sampler.c:8-18; flags src/main.c:951-963)."""
from __future__ import annotations

import dataclasses
import time

M64 = (1 << 64) - 1


@dataclasses.dataclass
class SamplingParams:
    temp: float = 0.0              # <= 0: greedy argmax, first maximum wins
    top_p: float = 1.0             # 1.0: off
    top_k: int = 0                 # 0: off
    min_p: float = 0.0             # 0.0: off
    repeat_penalty: float = 1.0    # 1.0: off; applies to stochastic sampling only
    repeat_last_n: int = 64        # ring of recent tokens the penalty looks at
    seed: int = 0                  # 0: seeded from the clock
    max_new_tokens: int = 128
    ignore_eos: bool = False

    def validate(self) -> None:
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")
        if not 0.0 <= self.min_p:
            raise ValueError("min_p must be >= 0")
        if self.seed < 0 or self.seed > M64:
            raise ValueError("seed must fit 64 unsigned bits")


class XorShift128Plus:
    """The reference's generator: seeding constants and 16 warm-up draws of src/sampler.c:33-45,
    step of :20-27, uniform = float32(next >> 11) * 2^-53 of :29-31."""

    def __init__(self, seed: int):
        if seed == 0:
            seed = time.monotonic_ns() & M64
        self.s0 = (seed ^ 0x8A5CD789635D2DFF) & M64
        self.s1 = (((seed + 0x9E3779B97F4A7C15) & M64) ^ 0x123456789ABCDEF0) & M64
        for _ in range(16):
            self.next_u64()

    def next_u64(self) -> int:
        s1, s0 = self.s0, self.s1
        self.s0 = s0
        s1 ^= (s1 << 23) & M64
        self.s1 = (s1 ^ s0 ^ (s1 >> 17) ^ (s0 >> 26)) & M64
        return (self.s1 + s0) & M64

    def uniform(self) -> float:
        import numpy as np
        return float(np.float32(np.float32(self.next_u64() >> 11) * np.float32(1.0 / 9007199254740992.0)))


class SamplerState:
    """What one request carries between draws: its generator and its ring of recent tokens
    (src/sampler.c:47-61, :83-90: capacity max(repeat_last_n or 64, 16))."""

    def __init__(self, params: SamplingParams):
        self.params = params
        self.rng = XorShift128Plus(params.seed)
        cap = params.repeat_last_n if params.repeat_last_n > 0 else 64
        self.cap = max(cap, 16)
        self.recent = [0] * self.cap
        self.head = 0
        self.count = 0

    def accept(self, token: int) -> None:
        self.recent[self.head] = token
        self.head = (self.head + 1) % self.cap
        self.count = min(self.count + 1, self.cap)
