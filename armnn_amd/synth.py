"""Seeded synthetic data with a self-defined generator, so every host produces the same bytes.

splitmix64 counter mode: element i of stream `seed` is mix(seed + (i+1)*GOLDEN).  Normal deviates use
Box-Muller in float64 on two such uniforms.  (std::normal_distribution / numpy's ziggurat are not
specified bit-exactly across library versions; this is.)
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _mix(z: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def u64(seed: int, n: int, stream: int = 0) -> np.ndarray:
    with np.errstate(over="ignore"):
        base = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + np.uint64(stream) * np.uint64(0xD1B54A32D192ED03)
        idx = np.arange(1, n + 1, dtype=np.uint64)
        return _mix(base + idx * _GOLDEN)


def uniform01(seed: int, n: int, stream: int = 0) -> np.ndarray:
    """float64 in [0,1) with 53 random bits."""
    return (u64(seed, n, stream) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform_int(seed: int, shape, lo: int, hi: int, dtype) -> np.ndarray:
    """Integers uniform in [lo, hi] inclusive."""
    n = int(np.prod(shape))
    span = hi - lo + 1
    v = (u64(seed, n) % np.uint64(span)).astype(np.int64) + lo
    return v.astype(dtype).reshape(shape)


def normal(seed: int, shape, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    n = int(np.prod(shape))
    u1 = uniform01(seed, n, stream=1)
    u2 = uniform01(seed, n, stream=2)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))      # 1-u1 in (0,1]
    z = r * np.cos(2.0 * np.pi * u2)
    return (mean + std * z).reshape(shape)


def int8_weights(seed: int, shape, std: float = 30.0) -> np.ndarray:
    """clip(round(N(0,std)), -127, 127) as int8."""
    return np.clip(np.rint(normal(seed, shape, 0.0, std)), -127, 127).astype(np.int8)


def int32_bias(seed: int, n: int, std: float = 500.0) -> np.ndarray:
    return np.rint(normal(seed, (n,), 0.0, std)).astype(np.int32)


def scales(seed: int, n: int, lo: float = 0.002, hi: float = 0.02) -> np.ndarray:
    return (lo + (hi - lo) * uniform01(seed, n, stream=3)).astype(np.float32)
