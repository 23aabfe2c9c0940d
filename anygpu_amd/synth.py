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


def normal_matrix_f16(seed: int, rows: int, cols: int, std: float = 1.0, slab_rows: int = 8192) -> np.ndarray:
    """N(0, std) as float16 [rows, cols], drawn in float32 in slabs of rows from one stream and rounded once: the large
    score matrices of the softmax configurations without a float32 copy of the whole."""
    out = np.empty((rows, cols), dtype=np.float16)
    gen = _gen(seed)
    for r0 in range(0, rows, slab_rows):
        blk = gen.standard_normal(size=(min(slab_rows, rows - r0), cols), dtype=np.float32)
        if std != 1.0:
            blk *= np.float32(std)
        out[r0:r0 + blk.shape[0]] = blk
    return out
