"""MI355X-native kernels behind anyGPU's matmul / softmax / causal conv1d entry points.

`anygpu_amd.capi` binds the C ABI (include/anygpu_hip.h), `anygpu_amd.ops` calls it on torch
device tensors, `anygpu_amd.build` compiles the native parts in-tree.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
