"""Seeded normal variates whose bits do not depend on where they are made: the host twin
of ``csrc/random_fill.hip``.

Element ``i`` of a tensor is a function of ``(seed_lo, seed_hi, i)`` alone.  32-bit integer
mixing gives two 24-bit uniforms; a Box-Muller step turns them into one normal variate.
The logarithm and the cosine are written out as single IEEE float32 operations (a 32-entry
table and four terms for the logarithm, polynomials on a quarter turn for the cosine), in
the same order as the kernel, which is compiled without fused multiply-adds: both give the
same bits.  numpy's float32 array operations round once per operation, which is all this
relies on.
"""

from __future__ import annotations

import math

import numpy as np

_U32 = np.uint32
_F32 = np.float32


def _f(bits: int) -> np.float32:
    return np.array([bits], dtype=np.uint32).view(np.float32)[0]


# float32(1 / c_i) and float32(ln c_i) for c_i = 1 + (i + 0.5) / 32
INV_C = np.array([1.0 / (1 + (i + 0.5) / 32) for i in range(32)], dtype=np.float64).astype(np.float32)
LN_C = np.array([math.log(1 + (i + 0.5) / 32) for i in range(32)], dtype=np.float64).astype(np.float32)

_HALF_PI = _f(0x3FC90FDB)
_LN2 = _f(0x3F317218)
_SIN = [_f(b) for b in (0xB2D7322B, 0x3638EF1D, 0xB9500D01, 0x3C088889, 0xBE2AAAAB)]  # -1/11! .. -1/3!
_COS = [_f(b) for b in (0x310F76C7, 0xB493F27E, 0x37D00D01, 0xBAB60B61, 0x3D2AAAAB, 0xBF000000)]  # 1/12! .. -1/2!
_LOG = [_f(b) for b in (0xBE800000, 0x3EAAAAAB, 0xBF000000)]  # -1/4, 1/3, -1/2


def _mix32(x: np.ndarray) -> np.ndarray:
    x = x ^ (x >> _U32(16))
    x = x * _U32(0x85EBCA6B)
    x = x ^ (x >> _U32(13))
    x = x * _U32(0xC2B2AE35)
    x = x ^ (x >> _U32(16))
    return x


def seed_key(seed_lo: int, seed_hi: int) -> np.uint32:
    with np.errstate(over="ignore"):
        hi = _mix32(np.array([(seed_hi + 0x9E3779B9) & 0xFFFFFFFF], dtype=np.uint32))
        return _mix32(np.array([seed_lo & 0xFFFFFFFF], dtype=np.uint32) ^ hi)[0]


def standard_normal(seed_lo: int, seed_hi: int, start: int, count: int) -> np.ndarray:
    """float32 variates of elements ``start .. start + count - 1``."""
    with np.errstate(over="ignore"):
        key = seed_key(seed_lo, seed_hi)
        index = np.arange(start, start + count, dtype=np.uint64)
        i_lo = (index & np.uint64(0xFFFFFFFF)).astype(np.uint32)
        i_hi = (index >> np.uint64(32)).astype(np.uint32)
        x = _mix32(key ^ i_lo)
        x = _mix32(x + i_hi + _U32(0x9E3779B9))
        k1 = _mix32(x ^ _U32(0x68E31DA4)) >> _U32(8)
        k2 = _mix32(x ^ _U32(0xB5297A4D)) >> _U32(8)

    # ln(u1), u1 = (k1 + 1) / 2^24 in (0, 1]
    u1 = (k1 + _U32(1)).astype(np.float32) * _f(0x33800000)
    ub = u1.view(np.uint32)
    e = ((ub >> _U32(23)).astype(np.int32) - np.int32(127)).astype(np.float32)
    mant = ub & _U32(0x7FFFFF)
    idx = (mant >> _U32(18)).astype(np.int64)
    m = (mant | _U32(0x3F800000)).view(np.float32)
    r = m * INV_C[idx]
    r = r - _F32(1.0)
    p = r * _LOG[0]
    p = p + _LOG[1]
    p = p * r
    p = p + _LOG[2]
    p = p * r
    p = p + _F32(1.0)
    p = p * r
    ln_u = LN_C[idx] + p
    e_ln2 = e * _LN2
    ln_u = e_ln2 + ln_u
    t = ln_u * _F32(-2.0)
    t = np.where(t > _F32(0.0), t, _F32(0.0)).astype(np.float32)
    radius = np.sqrt(t)

    # cos(2 pi k2 / 2^24): the quadrant from the two top bits, polynomials on [0, pi/2)
    quadrant = k2 >> _U32(22)
    f = (k2 & _U32(0x3FFFFF)).astype(np.float32) * _f(0x34800000)
    a = f * _HALF_PI
    a2 = a * a
    s = a2 * _SIN[0]
    for coeff in _SIN[1:]:
        s = s + coeff
        s = s * a2
    s = s + _F32(1.0)
    s = s * a
    c = a2 * _COS[0]
    for coeff in _COS[1:]:
        c = c + coeff
        c = c * a2
    c = c + _F32(1.0)
    cosine = np.where(quadrant == 1, -s, np.where(quadrant == 2, -c, np.where(quadrant == 3, s, c)))
    return (radius * cosine.astype(np.float32)).astype(np.float32)


def normal(seed_lo: int, seed_hi: int, count: int, mean: float, std: float, chunk: int = 1 << 22) -> np.ndarray:
    """``mean + std * z`` for ``count`` elements, float32, made chunk by chunk."""
    out = np.empty(count, dtype=np.float32)
    mean32, std32 = np.float32(mean), np.float32(std)
    for start in range(0, count, chunk):
        n = min(chunk, count - start)
        v = standard_normal(seed_lo, seed_hi, start, n) * std32
        out[start:start + n] = v + mean32
    return out
