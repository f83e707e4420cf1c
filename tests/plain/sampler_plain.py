"""Plain restatement of the reference sampler (src/sampler.c), in numpy float32.

Order (src/sampler.c:99-230): greedy if temp <= 0; else repetition penalty over
the ring of recent tokens -> maximum -> min-p filter on (l - max)/T -> sort
descending -> top-k -> softmax -> top-p with renormalisation -> one uniform draw,
first candidate with r <= cumulative probability.
"""
from __future__ import annotations

import math

import numpy as np

M64 = (1 << 64) - 1


class XorShift128Plus:
    """src/sampler.c:20-45: seeding constants, 16 warm-up draws, 53-bit uniform."""

    def __init__(self, seed: int):
        self.s = [(seed ^ 0x8A5CD789635D2DFF) & M64,
                  (((seed + 0x9E3779B97F4A7C15) & M64) ^ 0x123456789ABCDEF0) & M64]
        for _ in range(16):
            self.next()

    def next(self) -> int:
        s1, s0 = self.s[0], self.s[1]
        self.s[0] = s0
        s1 ^= (s1 << 23) & M64
        self.s[1] = (s1 ^ s0 ^ (s1 >> 17) ^ (s0 >> 26)) & M64
        return (self.s[1] + s0) & M64

    def uniform(self) -> np.float32:
        # (float)(x >> 11) * (1.0f / 2^53): the integer is rounded to float32 first.
        return np.float32(np.float32(self.next() >> 11) * np.float32(1.0 / 9007199254740992.0))


class PlainSampler:
    def __init__(self, temp=0.0, top_p=1.0, top_k=0, min_p=0.0, repeat_penalty=1.0,
                 repeat_last_n=64, seed=1):
        self.temp, self.top_p, self.top_k, self.min_p = temp, top_p, top_k, min_p
        self.repeat_penalty = repeat_penalty
        cap = repeat_last_n if repeat_last_n > 0 else 64      # src/sampler.c:56-57
        self.cap = max(cap, 16)
        self.recent = [0] * self.cap
        self.head = 0
        self.count = 0
        self.rng = XorShift128Plus(seed)

    def accept(self, tok: int):                                # src/sampler.c:83-90
        self.recent[self.head] = tok
        self.head = (self.head + 1) % self.cap
        self.count = min(self.count + 1, self.cap)

    def sample(self, logits: np.ndarray) -> int:
        logits = np.asarray(logits, dtype=np.float32)
        V = logits.shape[0]
        if self.temp <= 0.0:                                   # :103-113, first maximum wins
            best = int(np.argmax(logits))
            self.accept(best)
            return best
        l = logits.copy()
        rp = np.float32(self.repeat_penalty)
        if self.repeat_penalty > 1.0 and self.count > 0:       # :135-143, once per ring entry
            for k in range(self.count):
                t = self.recent[k]
                if 0 <= t < V:
                    l[t] = l[t] / rp if l[t] > 0 else l[t] * rp
        mx = l.max()
        inv_t = np.float32(1.0) / np.float32(self.temp)
        scaled = (l - mx) * inv_t
        lo = np.float32(-1e30)
        if 0.0 < self.min_p < 1.0:                             # :151-166
            lo = np.float32(math.log(self.min_p))
        ids = np.nonzero(scaled >= lo)[0]
        vals = scaled[ids]
        order = np.argsort(-vals, kind="stable")               # :177, ties: lowest id first here
        ids, vals = ids[order], vals[order]
        if self.top_k > 0 and len(ids) > self.top_k:           # :180-182
            ids, vals = ids[:self.top_k], vals[:self.top_k]
        ex = np.exp(vals).astype(np.float32)                   # :185-195
        s = np.float32(0)
        for e in ex:
            s = np.float32(s + e)
        p = ex * (np.float32(1) / s if s > 0 else np.float32(1))
        active = len(p)
        if 0.0 < self.top_p < 1.0:                             # :198-214
            cum = np.float32(0)
            for i in range(len(p)):
                cum = np.float32(cum + p[i])
                if cum >= np.float32(self.top_p):
                    active = i + 1
                    break
            sub = np.float32(0)
            for i in range(active):
                sub = np.float32(sub + p[i])
            if sub > 0:
                p = p.copy()
                p[:active] = p[:active] * (np.float32(1) / sub)
        r = self.rng.uniform()                                 # :217-226
        cum = np.float32(0)
        chosen = int(ids[0])
        for i in range(active):
            cum = np.float32(cum + p[i])
            if r <= cum or i == active - 1:
                chosen = int(ids[i])
                break
        self.accept(chosen)
        return chosen
