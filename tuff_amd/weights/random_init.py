"""Random-weights mode: from a configuration and a seed to tensors, or to a model folder
(config.json + model.safetensors) that loads like any other.

Matrices, embeddings and conv taps are N(0, 0.02); norm weights are 1 + N(0, 0.01).

The generator is specified down to the bit, so that a seed means the same model wherever and in
whatever order its tensors are made (host or GPU, whole or in pieces, by this file or by another
program that follows the text below).  Element i (row-major) of the tensor called `name` under
`seed`:

  key   = mix(seed * GOLDEN + crc32(name))                        (64-bit, wrapping)
  a, b  = mix(key + (2 i + 1) * GOLDEN), mix(key + (2 i + 2) * GOLDEN)
          (draws 2 i + 1 and 2 i + 2 of a SplitMix64 generator whose state starts at key)
  u1    = ((a >> 11) + 1) * 2^-53   in (0, 1],     u2 = (b >> 11) * 2^-53   in [0, 1)
  z     = sqrt(-2 ln u1) * cos(2 pi u2)                           (Box-Muller, float64)
  value = 0.02 z  or  1 + 0.01 z  in float64, rounded to float32, then to the stored type
          (round to nearest even both times)

  mix(x): x ^= x >> 30; x *= 0xBF58476D1CE4E5B9; x ^= x >> 27; x *= 0x94D049BB133111EB; x ^= x >> 31
  GOLDEN = 0x9E3779B97F4A7C15

ln, cos and the square root are not a library's (two libraries differ in the last bit, for the
root too): they are the float64 operations + - * / in a fixed order, each rounded once (no fused
multiply-add):

  ln u:   u = m 2^e with m in [0.5, 1); if m < SQRT_HALF: m = 2 m, e = e - 1
          s = (m - 1) / (m + 1); t = s s
          p = 1/21; for k = 9, 8, ..., 0: p = p t + 1 / (2 k + 1)
          ln u = e LN2 + 2 (s p)
  sqrt q: q = m 2^e with m in [0.5, 1) (q = 0: m = 0, e = 0); if e is odd: m = m / 2, e = e + 1
          y = 0.3 + 0.7 m; five times: y = 0.5 (y + m / y)
          sqrt q = y 2^(e / 2)
  cos 2 pi u:  v = u if u <= 0.5 else 1 - u; w = v if v <= 0.25 else 0.5 - v  (sign - if v > 0.25)
          x = TWO_PI w; t = x x
          p = 1/24!; for k = 11, 10, ..., 0: p = c_k - p t, with c_k = 1 / (2 k)!
          (the alternating series 1 - t/2! + t^2/4! - ... + t^12/24!)
          cos = sign p
"""
from __future__ import annotations

import json
import math
import os
import zlib

import torch

from ..config.base import ModelConfig
from ..parts.base import WeightDecl
from .safetensors_io import write_safetensors

STD_MATRIX = 0.02
STD_NORM = 0.01

GOLDEN = 0x9E3779B97F4A7C15
MIX1 = 0xBF58476D1CE4E5B9
MIX2 = 0x94D049BB133111EB
MASK64 = (1 << 64) - 1
SQRT_HALF = 0.7071067811865476
LN2 = 0.6931471805599453
TWO_PI = 6.283185307179586
LN_TERMS = 10                                   # 1/(2k+1) for k = 0..10
COS_TERMS = 12                                  # 1/(2k)! for k = 0..12
SQRT_STEPS = 5
POWERS = 32                                     # 2^(e/2) of -2 ln u1 lies within 2^-27 .. 2^4

CHUNK = {"cpu": 1 << 21, "cuda": 1 << 25}        # elements made at a time


def _mix_int(x: int) -> int:
    x &= MASK64
    x ^= x >> 30
    x = (x * MIX1) & MASK64
    x ^= x >> 27
    x = (x * MIX2) & MASK64
    x ^= x >> 31
    return x


def tensor_key(seed: int, name: str) -> int:
    return _mix_int((int(seed) & MASK64) * GOLDEN + zlib.crc32(name.encode()))


def _i64(x: int) -> int:
    """The 64-bit pattern x as the signed number that torch's int64 holds."""
    x &= MASK64
    return x - (1 << 64) if x >> 63 else x


def _shr(x: torch.Tensor, k: int) -> torch.Tensor:
    """Logical shift right of 64-bit patterns held as int64."""
    return (x >> k) & ((1 << (64 - k)) - 1)


def _mix(x: torch.Tensor) -> torch.Tensor:
    x = x ^ _shr(x, 30)
    x = x * _i64(MIX1)
    x = x ^ _shr(x, 27)
    x = x * _i64(MIX2)
    return x ^ _shr(x, 31)


def normal_deviates(key: int, start: int, count: int, device="cpu") -> torch.Tensor:
    """z of the elements start .. start + count - 1 of the stream `key`, float64 on `device`."""
    i = torch.arange(start, start + count, dtype=torch.int64, device=device)
    base = i * _i64(2 * GOLDEN) + _i64(key)                          # key + 2 i GOLDEN
    a = _mix(base + _i64(GOLDEN))
    b = _mix(base + _i64(2 * GOLDEN))
    del i, base
    u1 = (_shr(a, 11) + 1).to(torch.float64) * 2.0 ** -53
    u2 = _shr(b, 11).to(torch.float64) * 2.0 ** -53
    del a, b
    # ln u1
    m, e = torch.frexp(u1)
    low = m < SQRT_HALF
    m = torch.where(low, m * 2.0, m)
    e = torch.where(low, e - 1, e).to(torch.float64)
    s = (m - 1.0) / (m + 1.0)
    t = s * s
    p = torch.full_like(t, 1.0 / (2 * LN_TERMS + 1))
    for k in range(LN_TERMS - 1, -1, -1):
        p = p * t + 1.0 / (2 * k + 1)
    ln_u = e * LN2 + 2.0 * (s * p)
    del m, e, low, s, t, u1
    # the square root of q = -2 ln u1 by Newton's iteration from a line
    m, e = torch.frexp(-2.0 * ln_u)
    odd = (e & 1) == 1
    m = torch.where(odd, m * 0.5, m)
    half = (torch.where(odd, e + 1, e) >> 1).to(torch.int64)
    y = 0.3 + 0.7 * m
    for _ in range(SQRT_STEPS):
        y = 0.5 * (y + m / y)
    powers = torch.tensor([2.0 ** h for h in range(-POWERS, POWERS)], dtype=torch.float64, device=device)
    r = y * powers[half + POWERS]
    del m, e, odd, half, y, p, ln_u
    # cos(2 pi u2)
    v = torch.where(u2 <= 0.5, u2, 1.0 - u2)
    neg = v > 0.25
    w = torch.where(neg, 0.5 - v, v)
    x = TWO_PI * w
    t = x * x
    p = torch.full_like(t, 1.0 / math.factorial(2 * COS_TERMS))
    for k in range(COS_TERMS - 1, -1, -1):
        p = 1.0 / math.factorial(2 * k) - p * t
    c = torch.where(neg, -p, p)
    return r * c


def random_tensor(decl: WeightDecl, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    if decl.init not in ("norm", "normal"):
        raise ValueError(f"tensor '{decl.name}': unknown init '{decl.init}'")
    shape = tuple(int(n) for n in decl.shape)
    n = math.prod(shape)
    key = tensor_key(seed, decl.name)
    out = torch.empty(n, dtype=dtype, device=device)
    chunk = CHUNK["cuda" if torch.device(device).type == "cuda" else "cpu"]
    for start in range(0, n, chunk):
        count = min(chunk, n - start)
        z = normal_deviates(key, start, count, device)
        z = 1.0 + STD_NORM * z if decl.init == "norm" else STD_MATRIX * z
        out[start:start + count] = z.to(torch.float32).to(dtype)
    return out.view(shape)


def random_weights(decls: list[WeightDecl], seed: int, run_dtype: torch.dtype, device,
                   stored_dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    """Tensors made on `device` directly: rounded to `stored_dtype` as a file would hold them,
    then kept in the type a run of `run_dtype` keeps them in.  The same values, bit for bit, as
    a folder that write_random_model() wrote with this seed and stored type holds."""
    from .loader import target_dtype
    out = {}
    for d in decls:
        t = random_tensor(d, seed, stored_dtype, device)
        out[d.name] = t.to(target_dtype(stored_dtype, run_dtype)).contiguous()
    return out


def write_random_model(cfg: ModelConfig, out_dir: str, seed: int,
                       dtype: torch.dtype = torch.bfloat16, device=None) -> str:
    """Writes config.json and model.safetensors for `cfg` into out_dir and returns out_dir.
    device: where the values are computed (the same bits anywhere); default: a GPU if one is
    visible, else the host."""
    from ..models.registry import build_model
    if device is None:
        device = "cuda:0" if torch.cuda.is_available() else "cpu"
    model = build_model(cfg)
    decls = {d.name: d for d in model.weight_decls()}
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f, indent=2)
    write_safetensors(
        os.path.join(out_dir, "model.safetensors"),
        [(d.name, tuple(d.shape), dtype) for d in decls.values()],
        lambda name: random_tensor(decls[name], seed, dtype, device).cpu(),
        metadata={"format": "pt", "seed": seed})
    return out_dir
