"""Seeded synthetic inputs for the benchmark configurations.

One generator everywhere (tests, smoke, bench): SplitMix64 over a counter,
mapped to floats as  lo + (u >> 40) * 2^-24 * (hi - lo)  computed in f32, so a
value depends only on (seed, index) and any slice can be generated alone.
"""
from __future__ import annotations

import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed: int, n: int, offset: int = 0) -> np.ndarray:
    """n 64-bit outputs of SplitMix64 for state values seed + (offset+i+1)*gamma."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def unit_f32(seed: int, n: int, offset: int = 0) -> np.ndarray:
    """Uniform in [0, 1): 24 random bits times 2^-24, exact in f32."""
    return (splitmix64(seed, n, offset) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)


def uniform_f32(seed: int, n: int, lo: float, hi: float, offset: int = 0) -> np.ndarray:
    u = unit_f32(seed, n, offset)
    return (np.float32(lo) + u * np.float32(hi - lo)).astype(np.float32)


def normal_f32(seed: int, n: int, offset: int = 0) -> np.ndarray:
    """Standard normal by Box-Muller on two uniform streams (f64 math, rounded to f32)."""
    u1 = (splitmix64(seed, n, offset) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    u2 = (splitmix64(seed ^ 0x5851F42D4C957F2D, n, offset) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    return (r * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def uniform_f16_bits(seed: int, n: int, lo: float, hi: float, offset: int = 0) -> np.ndarray:
    """Uniform f32 values rounded to nearest-even f16; returned as raw uint16 bits."""
    return uniform_f32(seed, n, lo, hi, offset).astype(np.float16).view(np.uint16)
