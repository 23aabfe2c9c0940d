"""Shared test helpers: the error metrics the parity gates use."""
from __future__ import annotations

import numpy as np

FP16_ULP_AT_1 = 2.0 ** -10  # spacing of binary16 in [1, 2)


def scaled_rel_err(actual: np.ndarray, ref: np.ndarray, floor) -> float:
    """max_i |a_i - r_i| / (|r_i| + s): relative error with a scale floor s (scalar or
    broadcastable array), so that elements that are tiny by cancellation or underflow are
    judged against the typical output magnitude rather than against themselves."""
    a = np.asarray(actual, dtype=np.float64)
    r = np.asarray(ref, dtype=np.float64)
    s = np.asarray(floor, dtype=np.float64)
    return float(np.max(np.abs(a - r) / (np.abs(r) + s)))


def rel_l2(actual: np.ndarray, ref: np.ndarray) -> float:
    a = np.asarray(actual, dtype=np.float64)
    r = np.asarray(ref, dtype=np.float64)
    return float(np.sqrt(np.sum((a - r) ** 2) / np.sum(r * r + 1e-8)))


def sample_rows(n_rows: int, count: int, seed: int = 0) -> np.ndarray:
    """First rows, last rows and a seeded spread in between, sorted and unique."""
    rng = np.random.Generator(np.random.Philox(key=seed))
    edge = [r for r in (0, 1, 2, 3, n_rows - 2, n_rows - 1) if 0 <= r < n_rows]
    mid = rng.integers(0, n_rows, size=max(count - len(edge), 0)).tolist()
    return np.unique(np.array(edge + mid, dtype=np.int64))


def exact_int_product(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """a @ b for integer-valued operands as int64.  Computed in float64 (the BLAS path, which numpy's own int64
    product is not): every partial sum of integer products stays far below 2^53, so any order of summation is exact."""
    a64, b64 = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    assert float(np.abs(a64).max(initial=0.0)) * float(np.abs(b64).max(initial=0.0)) * a64.shape[-1] < 2.0 ** 52
    return (a64 @ b64).astype(np.int64)
