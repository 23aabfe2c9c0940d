""".dat tensor codec (numpy): little-endian int32 dim, int32 shape[dim], int32 dtype code, raw
row-major elements.  Same byte layout as the reference's srcs/io/dat_file.hpp:8-26 reader and
scripts/dnn_inspector/dnninspect/tensor.py:76-110 writer."""
from __future__ import annotations

import struct

import numpy as np

DTYPE_CODES = {np.dtype(np.int8): 0, np.dtype(np.int16): 1, np.dtype(np.int32): 2, np.dtype(np.float16): 4,
               np.dtype(np.float32): 5, np.dtype(np.float64): 6}
CODE_DTYPES = {v: k for k, v in DTYPE_CODES.items()}


def save_tensor(arr: np.ndarray, path) -> None:
    arr = np.ascontiguousarray(arr)
    with open(path, "wb") as f:
        f.write(struct.pack("<i", arr.ndim))
        for s in arr.shape:
            f.write(struct.pack("<i", s))
        f.write(struct.pack("<i", DTYPE_CODES[arr.dtype]))
        f.write(arr.astype(arr.dtype.newbyteorder("<"), copy=False).tobytes())


def load_tensor(path) -> np.ndarray:
    with open(path, "rb") as f:
        (dim,) = struct.unpack("<i", f.read(4))
        shape = struct.unpack("<" + "i" * dim, f.read(4 * dim))
        (code,) = struct.unpack("<i", f.read(4))
        dt = CODE_DTYPES[code]
        data = np.frombuffer(f.read(), dtype=dt.newbyteorder("<"))
    return data.reshape(shape).astype(dt)
