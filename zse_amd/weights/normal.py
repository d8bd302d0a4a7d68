"""The random-weights function on the host: the very values the device kernel makes.

``zk_fill_normal`` (csrc/elementwise.hip) draws Normal(mean, std) values as a pure function of
(seed, stream, element index): a 64-bit mix of the three gives two 24-bit integers, Box-Muller
turns them into two values.  Its logarithm, sine and cosine are short sums of single,
correctly rounded float32 operations in a fixed order (no library function, no fused
multiply-add); this module does the same operations in the same order with NumPy float32
arrays, so host and device agree bit for bit, in float32 and after rounding to bfloat16.  A
model of any size made on the device can therefore be made again on the host, whole or one
tensor at a time.  The reference has nothing of the kind (random values appear only in its
adapter tests, orchestrator/lora_manager.py:157).
"""
from __future__ import annotations

import zlib

import numpy as np

_U = np.uint64
_F = np.float32


def _mix64(z: np.ndarray) -> np.ndarray:
    z = z + _U(0x9E3779B97F4A7C15)
    z = (z ^ (z >> _U(30))) * _U(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> _U(27))) * _U(0x94D049BB133111EB)
    return z ^ (z >> _U(31))


def stream_of(name: str) -> int:
    """The stream number of a tensor: a checksum of its name (without a leading ``model.``)."""
    return zlib.crc32(name.encode())


def _log_u24(k: np.ndarray) -> np.ndarray:
    """ln(k / 2^24) for integers k in [1, 2^24], as exact_log_u24 on the device."""
    e = np.floor(np.log2(k.astype(np.float64))).astype(np.int64)          # exact for k < 2^53
    m = (k.astype(np.float64) / np.exp2(e.astype(np.float64))).astype(_F)  # k / 2^e is exact in float32
    big = m > _F(1.41421354)
    m = np.where(big, m * _F(0.5), m)
    e = e + big
    s = (m - _F(1.0)) / (m + _F(1.0))
    s2 = s * s
    p = np.full_like(s2, _F(0.111111112))
    for c in (0.142857149, 0.2, 0.333333343, 1.0):
        p = p * s2 + _F(c)
    lm = (_F(2.0) * s) * p
    return (e - 24).astype(_F) * _F(0.693147182) + lm


def _sincos_u24(j: np.ndarray):
    """sin and cos of 2 pi j / 2^24 for integers j in [0, 2^24), as exact_sincos_u24."""
    q = j >> _U(22)
    r = (j & _U(0x3FFFFF)).astype(np.int64)
    fold = r > 0x200000
    r = np.where(fold, 0x400000 - r, r)
    x = r.astype(_F) * _F(3.74507039e-07)
    x2 = x * x
    ps = np.full_like(x2, _F(2.75573188e-06))
    for c in (-1.98412701e-04, 8.33333377e-03, -1.66666672e-01):
        ps = ps * x2 + _F(c)
    s0 = x + (x * x2) * ps
    pc = np.full_like(x2, _F(-2.75573188e-07))
    for c in (2.48015876e-05, -1.38888892e-03, 4.16666679e-02, -0.5):
        pc = pc * x2 + _F(c)
    c0 = _F(1.0) + x2 * pc
    s1 = np.where(fold, c0, s0)
    c1 = np.where(fold, s0, c0)
    sn = np.select([q == 0, q == 1, q == 2], [s1, c1, -s1], -c1)
    cs = np.select([q == 0, q == 1, q == 2], [c1, -s1, -c1], s1)
    return sn.astype(_F), cs.astype(_F)


def normal(n: int, seed: int, stream: int, mean: float = 0.0, std: float = 1.0,
           first: int = 0) -> np.ndarray:
    """Elements [first, first + n) of the tensor (seed, stream) as float32: the bits
    ``zk_fill_normal`` writes for the same arguments."""
    if n <= 0:
        return np.zeros(0, _F)
    p0, p1 = first // 2, (first + n + 1) // 2
    with np.errstate(over="ignore"):
        base = _mix64(np.array([(int(seed) ^ (int(stream) * 0xD1342543DE82EF95)) & 0xFFFFFFFFFFFFFFFF], _U))
        r = _mix64(base + np.arange(p0, p1, dtype=_U))
    k = (r >> _U(40)) + _U(1)
    j = (r >> _U(8)) & _U(0xFFFFFF)
    rad = np.sqrt(_F(-2.0) * _log_u24(k))
    sn, cs = _sincos_u24(j)
    out = np.empty(2 * (p1 - p0), _F)
    out[0::2] = _F(mean) + _F(std) * (rad * cs)
    out[1::2] = _F(mean) + _F(std) * (rad * sn)
    lo = first - 2 * p0
    return out[lo:lo + n]


def normal_tensor(shape, seed: int, name: str, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    n = 1
    for s in shape:
        n *= int(s)
    return normal(n, seed, stream_of(name), mean, std).reshape(shape)
