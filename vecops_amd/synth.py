"""Seeded synthetic operands for the matmul path.

One counter-based 64-bit draw per element (splitmix64 finaliser of
``seed * GOLDEN + index``), so any slice of any tensor can be regenerated
bit-for-bit on another host without carrying state.  No libm calls: the
normal generator is a 12-term Irwin-Hall sum, exact in fp64.
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def draws(seed: int, count: int, offset: int = 0) -> np.ndarray:
    """``count`` uint64 draws for element indices offset .. offset+count-1."""
    with np.errstate(over="ignore"):
        base = np.uint64(seed) * _GOLDEN
        idx = np.arange(offset, offset + count, dtype=np.uint64)
        return _mix(base + idx)


def unit(seed: int, count: int, offset: int = 0) -> np.ndarray:
    """fp64 uniform in [0, 1) with 24 random bits (exact in fp32)."""
    return (draws(seed, count, offset) >> np.uint64(40)).astype(np.float64) * (2.0 ** -24)


def uniform_pm1(seed: int, shape) -> np.ndarray:
    """fp32 uniform in [-1, 1)."""
    n = int(np.prod(shape))
    return (2.0 * unit(seed, n) - 1.0).astype(np.float32).reshape(shape)


def normal(seed: int, shape, sigma: float = 1.0) -> np.ndarray:
    """fp32 normal(0, sigma): sigma * (sum of 12 uniforms - 6)."""
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float64)
    step = 1 << 20
    for start in range(0, n, step):
        m = min(step, n - start)
        u = unit(seed, 12 * m, 12 * start).reshape(m, 12)
        out[start:start + m] = u.sum(axis=1) - 6.0
    return (sigma * out).astype(np.float32).reshape(shape)


def int8_sym(seed: int, shape) -> np.ndarray:
    """int8 uniform in [-127, 127]."""
    n = int(np.prod(shape))
    return ((draws(seed, n) % np.uint64(255)).astype(np.int64) - 127).astype(np.int8).reshape(shape)


def scales(seed: int, shape) -> np.ndarray:
    """Positive fp32 scales 2^-7 * (1 + u)."""
    n = int(np.prod(shape))
    return ((2.0 ** -7) * (1.0 + unit(seed, n))).astype(np.float32).reshape(shape)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bits, round to nearest even, NaN -> 0x7fc0 (host helper for inputs)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    with np.errstate(over="ignore"):
        rounded = ((bits + (((bits >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF))) >> np.uint32(16))
    out = rounded.astype(np.uint16)
    out[np.isnan(x)] = 0x7FC0
    return out


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)
