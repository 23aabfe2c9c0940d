"""ctypes binding of libanygpu_hip.so (the C ABI declared in include/anygpu_hip.h).

The library is looked up in-tree only (anygpu_amd/lib/).  There is no fallback of any kind: if
the shared object is missing or a symbol cannot be resolved, loading raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libanygpu_hip.so"

ANYGPU_OK = 0
ANYGPU_ERR_NULL_POINTER = -1
ANYGPU_ERR_BAD_SHAPE = -2
ANYGPU_ERR_BAD_STRIDE = -3
ANYGPU_ERR_UNSUPPORTED = -4
ANYGPU_ERR_TOO_LARGE = -5
ANYGPU_ERR_SCRATCH_TOO_SMALL = -6
DECODE_STATIC_SCRATCH_BYTES = 8 * 1024 * 1024
WORKSPACE_BYTES = 64 * 1024 * 1024
WORKSPACE_MAX_BYTES = 1024 * 1024 * 1024
MAX_OWN_WORKSPACES = 8

A_ROW_MAJOR = 0
A_COL_MAJOR = 1
B_ROW_MAJOR = 0
B_COL_MAJOR = 1

# name -> (restype, argtypes); one entry per declaration in include/anygpu_hip.h
SIGNATURES = {
    "anygpu_hip_abi_version": (c_int, []),
    "anygpu_hip_target": (c_char_p, []),
    "anygpu_hip_error_string": (c_char_p, [c_int]),
    "anygpu_set_workspace": (c_int, [c_void_p, c_void_p, c_int64]),
    "anygpu_release_workspaces": (c_int, []),
    "anygpu_gemm_f16_f32acc": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                       c_int64, c_int64, c_int64, c_int, c_void_p]),
    "anygpu_gemm_f16_f32acc_bias": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                            c_int64, c_int64, c_int64, c_int, c_void_p]),
    "anygpu_gemm_f16_f32acc_softcap": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                               c_int64, c_int64, c_int64, c_int, c_float, c_void_p]),
    "anygpu_gemm_f16_f32acc_gelu_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                                c_int64, c_int64, c_int64, c_int, c_void_p]),
    "anygpu_gemm_f16_f32acc_probe": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                             c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p]),
    "anygpu_stream_probe": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int64, c_void_p]),
    "anygpu_gemm_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                c_int64, c_int64, c_int64, c_int, c_int, c_void_p]),
    "anygpu_gemm_f32_softcap": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                        c_int64, c_int64, c_int64, c_int, c_float, c_void_p]),
    "anygpu_gemm_f32_gelu_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                         c_int64, c_int64, c_int64, c_int, c_void_p]),
    "anygpu_gemm_f16_f32acc_batched": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                               c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                               c_int, c_void_p]),
    "anygpu_gemm_f32_batched": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                        c_int, c_int, c_void_p]),
    "anygpu_softmax_rows_masked_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                               c_int64, c_float, c_float, c_void_p]),
    "anygpu_softmax_rows_masked_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                               c_int64, c_float, c_float, c_void_p]),
    "anygpu_softmax_rows_f16": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                        c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_softmax_rows_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                        c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_causal_conv1d_silu_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "anygpu_causal_conv1d_silu_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "anygpu_causal_conv1d_silu_update_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                     c_int64, c_int64, c_int64, c_void_p]),
    "anygpu_causal_conv1d_silu_update_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                     c_int64, c_int64, c_int64, c_void_p]),
    "anygpu_sdp_attention_fwd_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                             c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_sdp_attention_fwd_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                             c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_sdp_attention_fwd_masked_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                    c_int64, c_int64, c_float, c_float, c_void_p]),
    "anygpu_sdp_attention_fwd_masked_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                    c_int64, c_int64, c_float, c_float, c_void_p]),
    "anygpu_sdp_attention_decode_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int64]),
    "anygpu_sdp_attention_decode_f32_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int64]),
    "anygpu_sdp_attention_decode_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                                c_int64, c_int64, c_int64, c_int64, c_int64,
                                                c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_sdp_attention_decode_f16_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                                       c_int64, c_int64, c_int64, c_int64, c_int64,
                                                       c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_sdp_attention_decode_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                                c_int64, c_int64, c_int64, c_int64, c_int64,
                                                c_float, c_float, c_int, c_int64, c_void_p]),
    "anygpu_gated_rmsnorm_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_int, c_void_p]),
    "anygpu_gated_rmsnorm_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_int, c_void_p]),
}

_lib = None


class AnyGpuError(RuntimeError):
    """A C ABI call returned a non-zero code."""

    def __init__(self, fn: str, code: int, text: str):
        super().__init__(f"{fn} failed with code {code}: {text}")
        self.code = code


def load() -> ctypes.CDLL:
    """Load the kernel library and bind every declared symbol.  Raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or python anygpu_amd/build.py) first. There is no CPU fallback.")
    # One HIP runtime per process: PyTorch wheels carry their own libamdhip64 (same soname as the
    # system one).  If torch is going to be used for device memory it has to be loaded before this
    # library, so that both resolve to the single runtime already mapped; loaded the other way
    # round, torch maps a second runtime and streams / device state are no longer shared.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def error_string(code: int) -> str:
    return load().anygpu_hip_error_string(code).decode()


def check(fn: str, code: int) -> None:
    if code != ANYGPU_OK:
        raise AnyGpuError(fn, code, error_string(code))
