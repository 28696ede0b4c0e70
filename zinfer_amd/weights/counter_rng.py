"""The random-weights mode's one generator: a counter-based draw.  The value of an element
depends on (seed, tensor name, element index) alone, so a tensor can be drawn in any pieces, on
any machine, by the HIP kernel (`csrc/randinit.hip`) or by this numpy twin, to the same bits.

    key  = mix(seed XOR fnv1a64(name))
    z    = mix(key + (index + 1) * 0x9E3779B97F4A7C15)        (SplitMix64's finaliser)
    k1, k2 = high and low 32 bits of z
    gain:    1 + (k1 / 2^32 * 0.2 - 0.1)                                    U(0.9, 1.1)
    normal:  sqrt(-2 ln((k1 + 1) / 2^32)) * cos(2 pi k2 / 2^32) * std       Box-Muller

evaluated in 64-bit floats and rounded once to float32 (then, for bfloat16, to the nearest
even bfloat16).  The logarithm and the cosine are this file's own short sequences of +, -, *,
/ (each correctly rounded by IEEE 754, never contracted into a fused multiply-add), not a
library's, which is what makes the two implementations agree bit for bit.
"""
from __future__ import annotations

import numpy as np

MASK = (1 << 64) - 1
GOLDEN = 0x9E3779B97F4A7C15
MIX1 = 0xBF58476D1CE4E5B9
MIX2 = 0x94D049BB133111EB
KIND = {"normal": 0, "gain": 1, "zeros": 2}

LN2 = 0.6931471805599453
SQRT_HALF = 0.7071067811865476
TWO_PI_OVER_2_32 = 6.283185307179586 / 4294967296.0
# ln m = 2 f (1 + f^2/3 + f^4/5 + ...), f = (m - 1) / (m + 1); |f| <= 0.1716 needs 12 terms
LOG_COEFFS = tuple(1.0 / (2 * k + 1) for k in range(12))
# Taylor series on [0, pi/4]: sin x = x (1 - x^2/3! + ...), cos x = 1 - x^2/2! + ...
SIN_COEFFS = (1.0, -1.0 / 6, 1.0 / 120, -1.0 / 5040, 1.0 / 362880, -1.0 / 39916800,
              1.0 / 6227020800, -1.0 / 1307674368000, 1.0 / 355687428096000)
COS_COEFFS = (1.0, -1.0 / 2, 1.0 / 24, -1.0 / 720, 1.0 / 40320, -1.0 / 3628800,
              1.0 / 479001600, -1.0 / 87178291200, 1.0 / 20922789888000)


def fnv1a64(text: str) -> int:
    h = 0xCBF29CE484222325
    for b in text.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & MASK
    return h


def mix64(z: int) -> int:
    z = ((z ^ (z >> 30)) * MIX1) & MASK
    z = ((z ^ (z >> 27)) * MIX2) & MASK
    return z ^ (z >> 31)


def tensor_key(seed: int, name: str) -> int:
    return mix64((int(seed) & MASK) ^ fnv1a64(name))


def _horner(coeffs, s: np.ndarray) -> np.ndarray:
    acc = np.full_like(s, coeffs[-1])
    for c in reversed(coeffs[:-1]):
        acc = acc * s + c
    return acc


_PIECE = 1 << 14     # the temporaries of a piece stay in the cache: several times faster


def draw(key: int, start: int, count: int, kind: str, std: float = 0.02) -> np.ndarray:
    """Elements ``start .. start + count`` of the tensor with ``key``, as float32."""
    if kind == "zeros":
        return np.zeros((count,), dtype=np.float32)
    if kind not in KIND:
        raise ValueError(f"unknown kind of draw {kind!r}")
    out = np.empty((count,), dtype=np.float32)
    for lo in range(0, count, _PIECE):
        n = min(_PIECE, count - lo)
        out[lo:lo + n] = _draw_piece(key, start + lo, n, kind, std)
    return out


def _draw_piece(key: int, start: int, count: int, kind: str, std: float) -> np.ndarray:
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z = np.uint64(key) + idx * np.uint64(GOLDEN)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(MIX1)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(MIX2)
        z = z ^ (z >> np.uint64(31))
    k1 = (z >> np.uint64(32)).astype(np.float64)
    k2 = (z & np.uint64(0xFFFFFFFF)).astype(np.int64)
    if kind == "gain":
        u = k1 * (1.0 / 4294967296.0)
        return (1.0 + (u * 0.2 - 0.1)).astype(np.float32)
    # ln((k1 + 1) / 2^32)
    m, e = np.frexp(k1 + 1.0)                    # exact: m in [0.5, 1)
    low = m < SQRT_HALF
    m = np.where(low, m * 2.0, m)
    e = np.where(low, e - 1, e)
    f = (m - 1.0) / (m + 1.0)
    ln = (e - 32).astype(np.float64) * LN2 + 2.0 * f * _horner(LOG_COEFFS, f * f)
    r = np.sqrt(-2.0 * ln)
    # cos(2 pi k2 / 2^32): the octant from the top three bits, the rest folded into [0, pi/4]
    octant = k2 >> 29
    frac = k2 & ((1 << 29) - 1)
    t = np.where((octant & 1) == 1, (1 << 29) - frac, frac).astype(np.float64)
    x = t * TWO_PI_OVER_2_32
    s = x * x
    sin_x = x * _horner(SIN_COEFFS, s)
    cos_x = _horner(COS_COEFFS, s)
    use_sin = ((octant + 1) & 2) != 0            # octants 1, 2, 5, 6
    negative = ((octant + 2) & 4) != 0           # octants 2, 3, 4, 5
    c = np.where(use_sin, sin_x, cos_x)
    c = np.where(negative, -c, c)
    return (r * c * std).astype(np.float32)


def to_bfloat16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> the 16 bits of the nearest-even bfloat16 (no NaN among the draws)."""
    b = x.view(np.uint32)
    return ((b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)) \
        .astype(np.uint16)
