"""Deterministic synthetic inputs for tests and benchmarks.

One splitmix64 stream per tensor: uniform floats are (x >> 40) * 2^-24 for f32 and
(x >> 11) * 2^-53 for f64, mapped to [lo, hi); integers are lo + x mod (hi - lo + 1).
The reference's benchmark draws from an unseeded CSPRNG (benchmark/gemm.zig:150-204), so
there is no reference stream to match; this generator only has to be reproducible.
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def splitmix64(seed: int, n: int) -> np.ndarray:
    """n outputs of splitmix64 started at `seed` (vectorised: state_i = seed + (i+1)*golden)."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + _GOLDEN * (np.arange(1, n + 1, dtype=np.uint64))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform(seed: int, shape, dtype, lo: float = -1.0, hi: float = 1.0) -> np.ndarray:
    dtype = np.dtype(dtype)
    n = int(np.prod(shape))
    x = splitmix64(seed, n)
    if dtype == np.float32:
        u = (x >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    else:
        u = (x >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    out = (dtype.type(lo) + u * dtype.type(hi - lo)).astype(dtype)
    return out.reshape(shape)


def normal(seed: int, shape, dtype) -> np.ndarray:
    """Standard normal values (Box-Muller on two splitmix64 streams, evaluated in float64)."""
    n = int(np.prod(shape))
    u1 = 1.0 - uniform(seed, (n,), np.float64, 0.0, 1.0)  # (0, 1]
    u2 = uniform(seed ^ 0x5A5A5A5A5A5A5A5A, (n,), np.float64, 0.0, 1.0)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return z.astype(dtype).reshape(shape)


def integers(seed: int, shape, dtype, lo: int, hi: int) -> np.ndarray:
    """Uniform integers in [lo, hi] of `dtype` (values are reduced into the dtype's range)."""
    dtype = np.dtype(dtype)
    n = int(np.prod(shape))
    x = splitmix64(seed, n)
    span = np.uint64(hi - lo + 1)
    vals = (x % span).astype(np.int64) + np.int64(lo)
    return vals.astype(dtype).reshape(shape)


def config_seed(config: int, tensor_index: int) -> int:
    return 0x5EED0000 + config * 16 + tensor_index
