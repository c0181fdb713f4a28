"""Seeded normal values from a counter, on the CPU: the twin of csrc/kernels/random_fill.hip.

Element i of a tensor depends on (key, i) alone: splitmix64's (i // 2 + 1)-th output from state
`key` gives two 24-bit uniforms, Box-Muller turns them into two normal values, the cosine's for
element 2p and the sine's for element 2p + 1.  The logarithm
and the cosine are polynomials of float32 additions, multiplications, one division and one
square root, each rounded on its own and in the order of the kernel, so that the CPU and the
GPU make the same bits.  The reference has no random-weights mode; this is what tests and
benchmarks run on.
"""
from __future__ import annotations

import numpy as np

_M = np.uint64(0xFFFFFFFFFFFFFFFF)
_F = np.float32


_BLOCK = 1 << 16        # elements made at a time: the temporaries of a block stay in the cache


def counter_normal(key: int, first: int, n: int, scale: float = 1.0, shift: float = 0.0,
                   out: np.ndarray = None) -> np.ndarray:
    """float32 [n]: normal(key, first + i) * scale + shift for i in range(n)."""
    if out is None:
        out = np.empty(n, dtype=_F)
    for lo in range(0, n, _BLOCK):
        hi = min(n, lo + _BLOCK)
        a, b = first + lo, first + hi                      # elements [a, b): pairs a // 2 .. (b + 1) // 2
        p0, p1 = a >> 1, (b + 1) >> 1
        even, odd = _pairs(key, p0, p1 - p0)
        both = np.empty(2 * (p1 - p0), dtype=_F)
        both[0::2], both[1::2] = even, odd
        out[lo:hi] = both[a - 2 * p0:b - 2 * p0] * _F(scale) + _F(shift)
    return out


def _pairs(key: int, first: int, n: int):
    """(even, odd): the two normal values of pairs first .. first + n - 1."""
    with np.errstate(over="ignore"):
        i = np.arange(first + 1, first + 1 + n, dtype=np.uint64)
        z = np.uint64(key & 0xFFFFFFFFFFFFFFFF) + i * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    k = (z >> np.uint64(40)).astype(np.uint32) + np.uint32(1)            # 1 .. 2^24
    b = ((z >> np.uint64(8)) & np.uint64(0xFFFFFF)).astype(np.uint32)
    # ln(k / 2^24) = (e - 24) ln 2 + ln m, k = m 2^e, m in [1/sqrt 2, sqrt 2)
    m, e = np.frexp(k.astype(_F))                                        # exact: k has at most 24 bits
    m = m * _F(2.0)
    e = e.astype(np.int32) - 1
    big = m > _F(1.41421354)
    m = np.where(big, m * _F(0.5), m)
    e = e + big.astype(np.int32)
    s = (m - _F(1.0)) / (m + _F(1.0))
    s2 = s * s
    p = np.full(n, 0.111111112, dtype=_F)
    for c in (0.142857149, 0.200000003, 0.333333343, 1.0):
        p = p * s2 + _F(c)
    ln_u = (e - 24).astype(_F) * _F(0.693147182) + (_F(2.0) * s) * p
    radius = np.sqrt(_F(-2.0) * ln_u)
    quarter = b >> np.uint32(22)
    t = (b & np.uint32(0x3FFFFF)).astype(_F) * _F(2.38418579e-07) * _F(1.57079637)
    t2 = t * t
    sn = np.full(n, -2.50521084e-08, dtype=_F)
    for c in (2.75573188e-06, -1.98412701e-04, 8.33333377e-03, -1.66666672e-01, 1.0):
        sn = sn * t2 + _F(c)
    sn = sn * t
    cs = np.full(n, 2.08767559e-09, dtype=_F)
    for c in (-2.75573192e-07, 2.48015876e-05, -1.38888892e-03, 4.16666679e-02, -0.5, 1.0):
        cs = cs * t2 + _F(c)
    c = np.where(quarter == 0, cs, np.where(quarter == 1, -sn, np.where(quarter == 2, -cs, sn)))
    sv = np.where(quarter == 0, sn, np.where(quarter == 1, cs, np.where(quarter == 2, -sn, -cs)))
    even, odd = radius * c, radius * sv
    assert even.dtype == _F and odd.dtype == _F
    return even, odd
