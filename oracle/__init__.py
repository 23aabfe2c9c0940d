"""numpy-facing wrapper of the CPU oracle (oracle/anygpu_oracle.c -> oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by the smoke check and by the CPU-baseline leg
of the benchmark; the product package (anygpu_amd) never imports it.  Each function forwards
to the C restatement of the reference's CPU implementation; see the header of
anygpu_oracle.c for the reference file:line each one follows and how it is pinned.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import POINTER, c_float, c_int, c_int32, c_int64, c_void_p
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "liboracle.so"

_lib = None


def build() -> Path:
    subprocess.run(["make", "-C", str(ORACLE_DIR)], check=True, stdout=subprocess.DEVNULL)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        _lib = ctypes.CDLL(str(LIB_PATH))
        _lib.oracle_max_threads.restype = c_int
    return _lib


def max_threads() -> int:
    return int(lib().oracle_max_threads())


def _ptr(a: np.ndarray) -> c_void_p:
    return c_void_p(a.ctypes.data)


def _elem_strides(a: np.ndarray) -> tuple[int, ...]:
    assert all(s % a.itemsize == 0 for s in a.strides)
    return tuple(s // a.itemsize for s in a.strides)


_MM = {np.dtype(np.float32): "oracle_tensor_mm_f32", np.dtype(np.float64): "oracle_tensor_mm_f64",
       np.dtype(np.int32): "oracle_tensor_mm_i32"}


def tensor_mm(lhs: np.ndarray, rhs: np.ndarray, rows: tuple[int, int] | None = None, threads: int = 1) -> np.ndarray:
    """res = lhs @ rhs the reference's way; strided views are honoured (a transposed view is a
    column-major operand).  `rows` = (begin, end) computes that row range only (others stay 0)."""
    assert lhs.ndim == 2 and rhs.ndim == 2 and lhs.shape[1] == rhs.shape[0], \
        "matrix multiplication requires compatible matrices"
    assert lhs.dtype == rhs.dtype and lhs.dtype in _MM
    m, k = lhs.shape
    n = rhs.shape[1]
    res = np.zeros((m, n), dtype=lhs.dtype)
    r0, r1 = rows if rows is not None else (0, m)
    ls, rs, os_ = _elem_strides(lhs), _elem_strides(rhs), _elem_strides(res)
    fn = getattr(lib(), _MM[lhs.dtype])
    fn.restype = None
    fn(_ptr(lhs), _ptr(rhs), _ptr(res), c_int64(m), c_int64(n), c_int64(k),
       c_int64(ls[0]), c_int64(ls[1]), c_int64(rs[0]), c_int64(rs[1]), c_int64(os_[0]), c_int64(os_[1]),
       c_int64(r0), c_int64(r1), c_int(threads))
    return res


def tensor_gemm(xt: np.ndarray, wt: np.ndarray, bt: np.ndarray, threads: int = 1) -> np.ndarray:
    assert xt.dtype == wt.dtype == bt.dtype == np.float32
    assert xt.ndim == 2 and wt.ndim == 2 and xt.shape[1] == wt.shape[0] and bt.shape == (wt.shape[1],)
    m, k = xt.shape
    n = wt.shape[1]
    res = np.zeros((m, n), dtype=np.float32)
    bt = np.ascontiguousarray(bt)
    xs, ws, os_ = _elem_strides(xt), _elem_strides(wt), _elem_strides(res)
    fn = lib().oracle_tensor_gemm_f32
    fn.restype = None
    fn(_ptr(xt), _ptr(wt), _ptr(bt), _ptr(res), c_int64(m), c_int64(n), c_int64(k),
       c_int64(xs[0]), c_int64(xs[1]), c_int64(ws[0]), c_int64(ws[1]), c_int64(os_[0]), c_int64(os_[1]),
       c_int64(0), c_int64(m), c_int(threads))
    return res


def tensor_softmax(x: np.ndarray, threads: int = 1) -> np.ndarray:
    assert x.ndim == 2, "softmax expects 2 dimensional tensors"
    assert x.dtype in (np.float32, np.float64)
    m, n = x.shape
    y = np.zeros((m, n), dtype=x.dtype)
    xs, ys = _elem_strides(x), _elem_strides(y)
    fn = lib().oracle_tensor_softmax_f32 if x.dtype == np.float32 else lib().oracle_tensor_softmax_f64
    fn.restype = None
    fn(_ptr(x), _ptr(y), c_int64(m), c_int64(n), c_int64(xs[0]), c_int64(xs[1]), c_int64(ys[0]), c_int64(ys[1]),
       c_int(threads))
    return y


def tensor_mul_scalar(x: np.ndarray, alpha: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    fn = lib().oracle_tensor_mul_scalar_f32
    fn.restype = None
    fn(_ptr(x), c_float(alpha), _ptr(y), c_int64(x.size))
    return y


def tensor_add(lhs: np.ndarray, rhs: np.ndarray) -> np.ndarray:
    lhs = np.ascontiguousarray(lhs, dtype=np.float32)
    rhs = np.ascontiguousarray(rhs, dtype=np.float32)
    assert lhs.shape == rhs.shape, "tensors are not elementwise compatible"
    y = np.empty_like(lhs)
    fn = lib().oracle_tensor_add_f32
    fn.restype = None
    fn(_ptr(lhs), _ptr(rhs), _ptr(y), c_int64(lhs.size))
    return y


def softcap(x: np.ndarray, cap: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    fn = lib().oracle_softcap_f32
    fn.restype = None
    fn(_ptr(x), c_float(cap), _ptr(y), c_int64(x.size))
    return y


def gemma_linear_softcap(x: np.ndarray, w: np.ndarray, cap: float, threads: int = 1) -> np.ndarray:
    """x [..., hsize], w [vsize, hsize] -> softcap(x w^T, cap) of shape [..., vsize]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    hsize = x.shape[-1]
    assert w.ndim == 2 and w.shape[1] == hsize, "hidden size should match for xt and wt"
    n = x.size // hsize if hsize else 0
    y = np.empty(x.shape[:-1] + (w.shape[0],), dtype=np.float32)
    fn = lib().oracle_gemma_linear_softcap_f32
    fn.restype = None
    fn(_ptr(x), _ptr(w), c_float(cap), _ptr(y), c_int64(n), c_int64(hsize), c_int64(w.shape[0]), c_int(threads))
    return y


def tensor_gelu_tanh(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    fn = lib().oracle_tensor_gelu_tanh_f32
    fn.restype = None
    fn(_ptr(x), _ptr(y), c_int64(x.size))
    return y


def tensor_mul(lhs: np.ndarray, rhs: np.ndarray) -> np.ndarray:
    lhs = np.ascontiguousarray(lhs, dtype=np.float32)
    rhs = np.ascontiguousarray(rhs, dtype=np.float32)
    assert lhs.shape == rhs.shape, "tensors are not elementwise compatible"
    y = np.empty_like(lhs)
    fn = lib().oracle_tensor_mul_f32
    fn.restype = None
    fn(_ptr(lhs), _ptr(rhs), _ptr(y), c_int64(lhs.size))
    return y


def gemma_mlp_upproj(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, threads: int = 1) -> np.ndarray:
    """x [..., hsize], w_gate / w_up [hsize, isize] -> gelu_tanh(x w_gate) * (x w_up) of shape [..., isize]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w_gate = np.ascontiguousarray(w_gate, dtype=np.float32)
    w_up = np.ascontiguousarray(w_up, dtype=np.float32)
    hsize = x.shape[-1]
    assert w_gate.shape == w_up.shape and w_gate.shape[0] == hsize
    n = x.size // hsize if hsize else 0
    y = np.empty(x.shape[:-1] + (w_gate.shape[1],), dtype=np.float32)
    fn = lib().oracle_gemma_mlp_upproj_f32
    fn.restype = None
    fn(_ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(y), c_int64(n), c_int64(hsize), c_int64(w_gate.shape[1]), c_int(threads))
    return y


def tensor_silu(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    fn = lib().oracle_tensor_silu_f32
    fn.restype = None
    fn(_ptr(x), _ptr(y), c_int64(x.size))
    return y


def tensor_rms_norm(x: np.ndarray, w: np.ndarray, eps: float, zero_centered: bool = False) -> np.ndarray:
    """RMS normalisation over the trailing axes that w spans."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    assert tuple(x.shape[x.ndim - w.ndim:]) == tuple(w.shape), "wt shape is incorrect"
    size = w.size
    y = np.empty_like(x)
    fn = lib().oracle_tensor_rms_norm_f32
    fn.restype = None
    fn(_ptr(x), _ptr(w), c_float(eps), c_int(int(zero_centered)), _ptr(y), c_int64(x.size // size if size else 0), c_int64(size))
    return y


def zamba_gated_rmsnorm(x: np.ndarray, z: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    z = np.ascontiguousarray(z, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    assert x.shape == z.shape and w.ndim == 1 and x.shape[-1] == w.shape[0]
    cols = w.shape[0]
    y = np.empty_like(x)
    fn = lib().oracle_zamba_gated_rmsnorm_f32
    fn.restype = None
    fn(_ptr(x), _ptr(z), _ptr(w), c_float(eps), _ptr(y), c_int64(x.size // cols if cols else 0), c_int64(cols))
    return y


def causal_conv1d_update(x: np.ndarray, state: np.ndarray, w: np.ndarray, b: np.ndarray):
    """One decode step.  x [batch, dims], state [batch, dims, width - 1] -> (y [batch, dims], new state)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    batch, dims = x.shape
    width = w.shape[1]
    assert w.shape[0] == dims and b.shape == (dims,) and state.shape == (batch, dims, width - 1)
    new_state = np.array(state, dtype=np.float32, order="C", copy=True)
    y = np.empty_like(x)
    fn = lib().oracle_causal_conv1d_update_f32
    fn.restype = None
    fn(_ptr(x), _ptr(new_state), _ptr(w), _ptr(b), _ptr(y), c_int64(batch), c_int64(dims), c_int64(width))
    return y, new_state


def causal_mask(q_len: int, k_len: int, diag: int = 0) -> np.ndarray:
    mask = np.empty((q_len, k_len), dtype=np.float32)
    fn = lib().oracle_causal_mask_f32
    fn.restype = None
    fn(_ptr(mask), c_int64(q_len), c_int64(k_len), c_int64(diag))
    return mask


def slide_mask(mask: np.ndarray, window: int) -> np.ndarray:
    """mask is [batch, 1, seq_len, mask_len] (or [seq_len, mask_len])."""
    m = np.ascontiguousarray(mask, dtype=np.float32)
    seq_len, mask_len = m.shape[-2], m.shape[-1]
    batch = m.size // (seq_len * mask_len)
    y = np.empty_like(m)
    fn = lib().oracle_slide_mask_f32
    fn.restype = None
    fn(_ptr(m), c_int32(window), c_int64(batch), c_int64(seq_len), c_int64(mask_len), _ptr(y))
    return y


def attention_softmax(x: np.ndarray, *, alpha: float = 1.0, softcap: float = 0.0, causal: bool = False,
                      window: int = 0, q_len: int = 0, diag: int = 0, row_index: np.ndarray | None = None,
                      threads: int = 1) -> np.ndarray:
    """scale -> (softcap) -> mask add -> softmax on the rows of a float32 [rows, cols] matrix,
    composed from the primitives above in the reference's call order.  With `row_index` only
    those rows are evaluated and returned, packed in that order."""
    assert x.ndim == 2 and x.dtype == np.float32 and x.strides[1] == 4
    rows, cols = x.shape
    if row_index is not None:
        idx = np.ascontiguousarray(row_index, dtype=np.int64)
        count = idx.size
        idx_ptr = idx.ctypes.data_as(POINTER(c_int64))
    else:
        idx, count, idx_ptr = None, rows, None
    y = np.zeros((count, cols), dtype=np.float32)
    fn = lib().oracle_attention_softmax_f32
    fn.restype = None
    fn(_ptr(x), _ptr(y), c_int64(rows), c_int64(cols), c_int64(x.strides[0] // 4), c_int64(q_len), c_int64(diag),
       c_float(alpha), c_float(softcap), c_int(int(causal)), c_int64(window), idx_ptr, c_int64(count), c_int(threads))
    return y


def sdp_attention_masked_scaled_fwd(q: np.ndarray, k: np.ndarray, v: np.ndarray, mask: np.ndarray, alpha: float,
                                    threads: int = 1) -> np.ndarray:
    """q [..., n_q, d], k and v [..., n_k, d] (same leading axes), mask [..., n_q, n_k] with leading 1s."""
    q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
    n_q, d = q.shape[-2:]
    n_k = k.shape[-2]
    assert k.shape[-1] == d and v.shape[-2:] == (n_k, d) and q.shape[:-2] == k.shape[:-2] == v.shape[:-2]
    m2 = np.ascontiguousarray(mask, dtype=np.float32).reshape(n_q, n_k)
    num = int(np.prod(q.shape[:-2], dtype=np.int64)) if q.ndim > 2 else 1
    y = np.zeros(q.shape, dtype=np.float32)
    fn = lib().oracle_sdp_attention_masked_scaled_fwd_f32
    fn.restype = None
    fn(_ptr(q), _ptr(k), _ptr(v), _ptr(m2), c_float(alpha), _ptr(y), c_int64(num), c_int64(n_q), c_int64(n_k),
       c_int64(d), c_int(threads))
    return y


def sdp_attention_rules(q: np.ndarray, k: np.ndarray, v: np.ndarray, *, alpha: float, softcap: float = 0.0,
                        causal: bool = False, window: int = 0, q_per_kv: int = 1,
                        query_index: np.ndarray | None = None, threads: int = 1) -> np.ndarray:
    """softmax(mask(softcap(alpha q k^T))) v with masks given as index rules, composed per head from tensor_mm,
    attention_softmax and tensor_mm in the call order of srcs/transformers/sdp.hpp:258-271.  q [heads, n_q, d],
    k and v [heads / q_per_kv, n_k, d]; the causal diagonal sits at n_k - n_q.  With `query_index` only those
    queries of every head are evaluated (result [heads, len(query_index), d])."""
    q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
    heads, n_q, d = q.shape
    n_k = k.shape[1]
    assert k.shape == v.shape and k.shape[0] * q_per_kv == heads and k.shape[2] == d
    idx = np.arange(n_q, dtype=np.int64) if query_index is None else np.ascontiguousarray(query_index, dtype=np.int64)
    out = np.zeros((heads, idx.size, d), dtype=np.float32)
    for h in range(heads):
        kh, vh = k[h // q_per_kv], v[h // q_per_kv]
        qk = tensor_mm(q[h][idx], kh.T, threads=threads)
        # row r of qk is query idx[r]: hand the softmax one-row matrices' worth of indices through q_len / diag
        p = np.empty_like(qk)
        for r, i in enumerate(idx):
            p[r] = attention_softmax(qk[r:r + 1], alpha=alpha, softcap=softcap, causal=causal, window=window,
                                     q_len=0, diag=int(i) + (n_k - n_q))[0]
        out[h] = tensor_mm(p, vh, threads=threads)
    return out


def tensor_causal_conv1d(xt: np.ndarray, wt: np.ndarray, bt: np.ndarray, rows: tuple[int, int] | None = None,
                         threads: int = 1) -> np.ndarray:
    assert xt.ndim == 3, "xt needs to be 3 dimensional"
    assert xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims"
    assert wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims"
    assert xt.dtype == wt.dtype == bt.dtype and xt.dtype in (np.float32, np.float64)
    assert xt.strides[2] == xt.itemsize and wt.strides[1] == wt.itemsize
    b, d, s = xt.shape
    y = np.zeros((b, d, s), dtype=xt.dtype)
    bt = np.ascontiguousarray(bt)
    xs, ys, ws = _elem_strides(xt), _elem_strides(y), _elem_strides(wt)
    r0, r1 = rows if rows is not None else (0, b * d)
    fn = lib().oracle_tensor_causal_conv1d_f32 if xt.dtype == np.float32 else lib().oracle_tensor_causal_conv1d_f64
    fn.restype = None
    fn(_ptr(xt), _ptr(wt), _ptr(bt), _ptr(y), c_int64(b), c_int64(d), c_int64(s), c_int64(wt.shape[1]),
       c_int64(xs[0]), c_int64(xs[1]), c_int64(ys[0]), c_int64(ys[1]), c_int64(ws[0]),
       c_int64(r0), c_int64(r1), c_int(threads))
    return y


def cvt_f16_to_f32(h: np.ndarray) -> np.ndarray:
    """The reference's half -> float up-cast, from the raw 16-bit patterns."""
    bits = np.ascontiguousarray(h).view(np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    fn = lib().oracle_cvt_f16_to_f32
    fn.restype = None
    fn(_ptr(bits), _ptr(out), c_int64(bits.size))
    return out


def _compare(name: str, actual: np.ndarray, expected: np.ndarray, tol: float) -> tuple[bool, float]:
    a = np.ascontiguousarray(actual, dtype=np.float32)
    e = np.ascontiguousarray(expected, dtype=np.float32)
    assert a.shape == e.shape
    worst = c_float(0.0)
    fn = getattr(lib(), name)
    fn.restype = c_int
    ok = fn(_ptr(a), _ptr(e), c_int64(a.size), c_float(tol), ctypes.byref(worst))
    return bool(ok), float(worst.value)


def compare_data_buffers(actual, expected, abs_tol: float = 0.001):
    return _compare("oracle_compare_abs_f32", actual, expected, abs_tol)


def compare_data_buffers_reldiff(actual, expected, rel_tol: float = 0.01):
    return _compare("oracle_compare_reldiff_f32", actual, expected, rel_tol)


def compare_data_buffers_l2(actual, expected, rel_l2: float = 0.01):
    return _compare("oracle_compare_l2_f32", actual, expected, rel_l2)
