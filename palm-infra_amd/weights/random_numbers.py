"""Counter-based normal random numbers, on the host, with the same bits as the device kernel
``palm_random_fill`` (csrc/weights_prep.hip).

Element ``i`` of a tensor is a function of ``(key, i)`` alone; the key is a hash of the seed and the tensor's
checkpoint name.  So a tensor does not depend on which other tensors a model has or in which order they are
made, a model folder and a model made on the device hold the same numbers, and layer ``k`` of a deep model is
layer ``k`` of a shallow one.  Every arithmetic step is one correctly rounded float32 operation (numpy's
elementwise float32 add, multiply, divide and square root are) or integer arithmetic, in the order in which
the kernel does them; see the formulas there.
"""
from __future__ import annotations

import hashlib

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1, _M2 = np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB)
_MASK = (1 << 64) - 1


def _f(hex_text: str) -> np.float32:
    return np.float32(float.fromhex(hex_text))


_SQRT2, _LN2, _TWO_PI, _HALF_SQRT = _f("0x1.6a09e6p+0"), _f("0x1.62e430p-1"), _f("0x1.921fb6p+2"), _f("0x1.6a09e6p-1")
_LN_SERIES = [_f("0x1.c71c72p-4"), _f("0x1.24924ap-3"), _f("0x1.99999ap-3"), _f("0x1.555556p-2"), np.float32(1.0)]
_SIN_SERIES = [_f("0x1.71de3ap-19"), _f("-0x1.a01a02p-13"), _f("0x1.111112p-7"), _f("-0x1.555556p-3"), np.float32(1.0)]
_COS_SERIES = [_f("0x1.a01a02p-16"), _f("-0x1.6c16c2p-10"), _f("0x1.555556p-5"), np.float32(-0.5), np.float32(1.0)]


def tensor_key(seed: int, name: str) -> int:
    """64 bits from the seed and the tensor's name (the name goes through SHA-256, so that similar names give
    unrelated keys)."""
    digest = hashlib.sha256(name.encode()).digest()
    x = (int.from_bytes(digest[:8], "little") ^ ((int(seed) * 0x9E3779B97F4A7C15) & _MASK)) & _MASK
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _MASK
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _MASK
    x ^= x >> 31
    return x


def _mix64(x: np.ndarray) -> np.ndarray:
    x = x ^ (x >> np.uint64(30))
    x = x * _M1
    x = x ^ (x >> np.uint64(27))
    x = x * _M2
    return x ^ (x >> np.uint64(31))


def _series(coefficients, t):
    p = np.full_like(t, coefficients[0])
    for c in coefficients[1:]:
        p = p * t + c
    return p


def standard_normal(key: int, first: int, count: int) -> np.ndarray:
    """Elements ``first .. first + count`` of the stream of ``key``, float32."""
    with np.errstate(over="ignore"):
        i = np.arange(first + 1, first + count + 1, dtype=np.uint64)
        h = _mix64(np.uint64(key) + i * _GOLDEN)
    a = (h >> np.uint64(41)).astype(np.uint32)
    b = ((h >> np.uint64(17)) & np.uint64(0xFFFFFF)).astype(np.uint32)
    u = (np.uint32(2) * a + np.uint32(1)).astype(np.float32) * np.float32(2.0 ** -24)
    bits = u.view(np.uint32)
    e = (bits >> np.uint32(23)).astype(np.int32) - np.int32(127)
    m = ((bits & np.uint32(0x7FFFFF)) | np.uint32(0x3F800000)).view(np.float32)
    big = m > _SQRT2
    m = np.where(big, m * np.float32(0.5), m)
    e = np.where(big, e + np.int32(1), e)
    s = (m - np.float32(1.0)) / (m + np.float32(1.0))
    p = _series(_LN_SERIES, s * s)
    ln_u = e.astype(np.float32) * _LN2 + (s * p) * np.float32(2.0)
    r = np.sqrt(np.float32(-2.0) * ln_u)
    octant, frac = b >> np.uint32(21), b & np.uint32(0x1FFFFF)
    x = (frac.astype(np.float32) * np.float32(2.0 ** -24)) * _TWO_PI
    x2 = x * x
    sin_x = x * _series(_SIN_SERIES, x2)
    cos_x = _series(_COS_SERIES, x2)
    diff, total = (cos_x - sin_x) * _HALF_SQRT, (cos_x + sin_x) * _HALF_SQRT
    c = np.select([octant == 0, octant == 1, octant == 2, octant == 3, octant == 4, octant == 5, octant == 6],
                  [cos_x, diff, -sin_x, -total, -cos_x, -diff, sin_x], default=total)
    return (r * c).astype(np.float32)


def normal(key: int, count: int, mean: float, std: float, chunk: int = 1 << 18) -> np.ndarray:
    """``count`` float32 values ``z * std + mean`` (a rounded product, then a rounded sum).  Made in pieces that stay
    in the processor's caches (some ten million values a second)."""
    out = np.empty((count,), dtype=np.float32)
    mean32, std32 = np.float32(mean), np.float32(std)
    for lo in range(0, count, chunk):
        n = min(chunk, count - lo)
        out[lo:lo + n] = standard_normal(key, lo, n) * std32 + mean32
    return out
