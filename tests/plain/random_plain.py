"""The random-weights generator restated in numpy from its specification (the docstring of
tuff_amd/weights/random_init.py), sharing no code with it: 64-bit patterns are numpy's unsigned
integers here (wrapping by definition), signed ones with masked shifts there.

The reference has no random-weights mode (it always loads a real checkpoint); the distribution,
N(0, 0.02) for matrices and 1 + N(0, 0.01) for norm weights, is the benchmark's own statement."""
import math
import zlib

import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def mix(x):
    x = x ^ (x >> np.uint64(30))
    x = x * np.uint64(0xBF58476D1CE4E5B9)
    x = x ^ (x >> np.uint64(27))
    x = x * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def key_of(seed: int, name: str) -> np.uint64:
    with np.errstate(over="ignore"):
        return mix(np.array([seed % 2 ** 64], dtype=np.uint64) * GOLDEN + np.uint64(zlib.crc32(name.encode())))[0]


def deviates(seed: int, name: str, n: int) -> np.ndarray:
    """z_0 .. z_{n-1} of the tensor `name`: standard normal deviates, float64."""
    with np.errstate(over="ignore"):
        key = key_of(seed, name)
        i = np.arange(n, dtype=np.uint64)
        a = mix(key + (np.uint64(2) * i + np.uint64(1)) * GOLDEN)
        b = mix(key + (np.uint64(2) * i + np.uint64(2)) * GOLDEN)
    u1 = ((a >> np.uint64(11)) + np.uint64(1)).astype(np.float64) * 2.0 ** -53
    u2 = (b >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    # ln u1 from + - * / alone
    m, e = np.frexp(u1)
    e = e.astype(np.float64)
    low = m < 0.7071067811865476
    m[low] *= 2.0
    e[low] -= 1.0
    s = (m - 1.0) / (m + 1.0)
    t = s * s
    p = np.full(n, 1.0 / 21)
    for k in range(9, -1, -1):
        p = p * t + 1.0 / (2 * k + 1)
    ln_u = e * 0.6931471805599453 + 2.0 * (s * p)
    # the root of q = -2 ln u1: Newton's iteration on the mantissa, the exponent halved
    m, e = np.frexp(-2.0 * ln_u)
    odd = e % 2 == 1
    m[odd] /= 2.0
    e[odd] += 1
    y = 0.3 + 0.7 * m
    for _ in range(5):
        y = 0.5 * (y + m / y)
    r = np.ldexp(y, e // 2)
    # cos 2 pi u2 from its series on [0, pi / 2]
    v = np.where(u2 <= 0.5, u2, 1.0 - u2)
    neg = v > 0.25
    w = np.where(neg, 0.5 - v, v)
    x = 6.283185307179586 * w
    t = x * x
    p = np.full(n, 1.0 / math.factorial(24))
    for k in range(11, -1, -1):
        p = 1.0 / math.factorial(2 * k) - p * t
    return r * np.where(neg, -p, p)


def to_bfloat16_bits(x32: np.ndarray) -> np.ndarray:
    """float32 -> the 16 bits of the nearest bfloat16 (ties to even); finite values only."""
    bits = x32.astype(np.float32).view(np.uint32)
    return ((bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def tensor_f32(seed: int, name: str, shape, init: str) -> np.ndarray:
    """The tensor as float32 (before the rounding to the stored type)."""
    z = deviates(seed, name, int(np.prod(shape)))
    v = 1.0 + 0.01 * z if init == "norm" else 0.02 * z
    return v.astype(np.float32).reshape(shape)
