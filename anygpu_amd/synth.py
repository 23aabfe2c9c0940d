"""Deterministic synthetic inputs (numpy, host side) for tests and the benchmark.

A counter-based generator (Philox) keyed by the seed gives the same stream on every host.
The second parameter of N(., .) is a standard deviation (torch.normal_(mean, std) convention).
"""
from __future__ import annotations

import numpy as np


def _gen(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(key=int(seed)))


def normal(seed: int, shape, std: float = 1.0, mean: float = 0.0, dtype=np.float32) -> np.ndarray:
    x = _gen(seed).standard_normal(size=shape, dtype=np.float32)
    if std != 1.0:
        x *= np.float32(std)
    if mean != 0.0:
        x += np.float32(mean)
    return x.astype(dtype, copy=False)


def uniform(seed: int, shape, lo: float = -1.0, hi: float = 1.0, dtype=np.float32) -> np.ndarray:
    x = _gen(seed).random(size=shape, dtype=np.float32)
    x = x * np.float32(hi - lo) + np.float32(lo)
    return x.astype(dtype, copy=False)


def integers(seed: int, shape, lo: int, hi: int, dtype=np.float32) -> np.ndarray:
    """Integer values in [lo, hi] stored in a floating type (exact sums, order independent)."""
    return _gen(seed).integers(lo, hi + 1, size=shape).astype(dtype)
