"""Thin Python callers of the C ABI on torch device tensors.

torch is used for device memory and the current stream only; every computation happens in
libanygpu_hip.so.  The function names follow the reference's operator API (tensor_mm,
tensor_gemm, tensor_softmax, tensor_causal_conv1d; srcs/ops/mm_ops.hpp, srcs/ops/softmax_ops.hpp,
srcs/fused/causal_conv1d.hpp), with the fused attention prologue and the B layout as the
additional keyword arguments the C ABI carries.
"""
from __future__ import annotations

import torch

from . import capi


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _check_device(*tensors: torch.Tensor) -> None:
    for t in tensors:
        _require(t.is_cuda, "anygpu ops take device tensors only (no CPU fallback)")


def set_workspace(workspace: torch.Tensor | None, stream: torch.cuda.Stream | None = None) -> None:
    """Hand the GEMM entry points a caller-owned K-split workspace for `stream` (default: the current stream), or take
    it back with None.  The tensor must stay alive while launches or graphs that used it can still run."""
    lib = capi.load()
    handle = (stream or torch.cuda.current_stream()).cuda_stream
    if workspace is None:
        capi.check("anygpu_set_workspace", lib.anygpu_set_workspace(handle, None, 0))
        return
    _check_device(workspace)
    _require(workspace.is_contiguous(), "the workspace must be dense")
    capi.check("anygpu_set_workspace", lib.anygpu_set_workspace(handle, workspace.data_ptr(), workspace.numel() * workspace.element_size()))


def release_workspaces() -> None:
    """Free every K-split workspace the library allocated itself and forget all registrations."""
    capi.check("anygpu_release_workspaces", capi.load().anygpu_release_workspaces())


def tensor_mm(lhs: torch.Tensor, rhs: torch.Tensor, out: torch.Tensor | None = None,
              b_layout: int = capi.B_ROW_MAJOR, a_layout: int = capi.A_ROW_MAJOR) -> torch.Tensor:
    """C = A @ B.  With a_layout == A_ROW_MAJOR lhs is [M, K] (rows may be padded: stride(0) >= K,
    stride(1) == 1); with A_COL_MAJOR (float32 only) lhs is the [K, M] storage of A.
    With b_layout == B_ROW_MAJOR rhs is [K, N]; with B_COL_MAJOR rhs is the [N, K] storage of B.
    float16 (fp32 accumulate) and float32 are supported."""
    _check_device(lhs, rhs)
    _require(lhs.dim() == 2 and rhs.dim() == 2, "matrix multiplication requires compatible matrices")
    _require(lhs.dtype == rhs.dtype, "operands must share a dtype")
    _require(lhs.stride(1) == 1 and rhs.stride(1) == 1, "innermost stride must be 1")
    m, k = lhs.shape if a_layout == capi.A_ROW_MAJOR else (lhs.shape[1], lhs.shape[0])
    if b_layout == capi.B_ROW_MAJOR:
        _require(rhs.shape[0] == k, "matrix multiplication requires compatible matrices")
        n = rhs.shape[1]
    else:
        _require(rhs.shape[1] == k, "matrix multiplication requires compatible matrices")
        n = rhs.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=lhs.dtype, device=lhs.device)
    _require(tuple(out.shape) == (m, n) and out.stride(1) == 1, "result mtx shape is wrong")
    lib = capi.load()
    lda = lhs.stride(0) if lhs.shape[0] > 1 else max(lhs.shape[1], 1)
    ldb = rhs.stride(0) if rhs.shape[0] > 1 else max(rhs.shape[1], 1)
    ldc = out.stride(0) if m > 1 else max(n, 1)
    if lhs.dtype == torch.float16:
        _require(a_layout == capi.A_ROW_MAJOR, "the fp16 GEMM takes a row-major left operand")
        rc = lib.anygpu_gemm_f16_f32acc(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), m, n, k,
                                        lda, ldb, ldc, b_layout, _stream_ptr())
        capi.check("anygpu_gemm_f16_f32acc", rc)
    elif lhs.dtype == torch.float32:
        rc = lib.anygpu_gemm_f32(lhs.data_ptr(), rhs.data_ptr(), None, out.data_ptr(), m, n, k,
                                 lda, ldb, ldc, a_layout, b_layout, _stream_ptr())
        capi.check("anygpu_gemm_f32", rc)
    else:
        raise TypeError("Unsupported data type")
    return out


def tensor_gemm(xt: torch.Tensor, wt: torch.Tensor, bt: torch.Tensor,
                b_layout: int = capi.B_ROW_MAJOR) -> torch.Tensor:
    """xt @ wt + bt (bias per output column), float32 or float16 (fp32 sums, bias added before the rounding)."""
    _check_device(xt, wt, bt)
    _require(xt.dim() == 2 and wt.dim() == 2, "matrix multiplication requires compatible matrices")
    _require(xt.dtype in (torch.float32, torch.float16) and wt.dtype == xt.dtype and bt.dtype == xt.dtype,
             "Unsupported data type")
    _require(xt.is_contiguous() and wt.is_contiguous() and bt.is_contiguous(), "dense operands expected")
    m, k = xt.shape
    n = wt.shape[1] if b_layout == capi.B_ROW_MAJOR else wt.shape[0]
    _require((wt.shape[0] if b_layout == capi.B_ROW_MAJOR else wt.shape[1]) == k,
             "matrix multiplication requires compatible matrices")
    _require(bt.numel() == n, "incorrect bias shape")
    out = torch.empty((m, n), dtype=xt.dtype, device=xt.device)
    if xt.dtype == torch.float16:
        rc = capi.load().anygpu_gemm_f16_f32acc_bias(xt.data_ptr(), wt.data_ptr(), bt.data_ptr(), out.data_ptr(), m, n, k,
                                                     max(k, 1), max(wt.shape[1], 1), max(n, 1), b_layout, _stream_ptr())
        capi.check("anygpu_gemm_f16_f32acc_bias", rc)
        return out
    rc = capi.load().anygpu_gemm_f32(xt.data_ptr(), wt.data_ptr(), bt.data_ptr(), out.data_ptr(), m, n, k,
                                     max(k, 1), max(wt.shape[1], 1), max(n, 1), capi.A_ROW_MAJOR, b_layout,
                                     _stream_ptr())
    capi.check("anygpu_gemm_f32", rc)
    return out


def tensor_gemma_linear_softcap(xt: torch.Tensor, wt: torch.Tensor, final_softcapping: float) -> torch.Tensor:
    """softcap(xt @ wt^T): xt [b, s, hidden], wt [vocab, hidden] -> [b, s, vocab], float32 or float16.

    Same contract as tensor_gemma_linear_softcap of the reference (srcs/models/gemma2/gemma_linsoftcap.hpp:12-41).
    """
    _check_device(xt, wt)
    _require(xt.dim() == 3, "xt should be 3 dim")
    _require(wt.dim() == 2 and xt.shape[2] == wt.shape[1], "hidden size should match for xt and wt")
    _require(xt.dtype in (torch.float32, torch.float16) and wt.dtype == xt.dtype, "Unsupported data types")
    _require(xt.is_contiguous() and wt.is_contiguous(), "dense operands expected")
    m, k, n = xt.shape[0] * xt.shape[1], xt.shape[2], wt.shape[0]
    out = torch.empty((xt.shape[0], xt.shape[1], n), dtype=xt.dtype, device=xt.device)
    if xt.dtype == torch.float16:
        rc = capi.load().anygpu_gemm_f16_f32acc_softcap(xt.data_ptr(), wt.data_ptr(), out.data_ptr(), m, n, k,
                                                        max(k, 1), max(k, 1), max(n, 1), capi.B_COL_MAJOR,
                                                        float(final_softcapping), _stream_ptr())
        capi.check("anygpu_gemm_f16_f32acc_softcap", rc)
        return out
    rc = capi.load().anygpu_gemm_f32_softcap(xt.data_ptr(), wt.data_ptr(), out.data_ptr(), m, n, k,
                                             max(k, 1), max(k, 1), max(n, 1), capi.B_COL_MAJOR,
                                             float(final_softcapping), _stream_ptr())
    capi.check("anygpu_gemm_f32_softcap", rc)
    return out


def mlp_gemma2_fused_upproj(xt: torch.Tensor, wt_gp: torch.Tensor, wt_up: torch.Tensor,
                            b_layout: int = capi.B_ROW_MAJOR) -> torch.Tensor:
    """gelu_tanh(xt @ wt_gp) * (xt @ wt_up): xt [..., hidden], weights [hidden, intermediate] (or [intermediate, hidden]
    with B_COL_MAJOR), float32 or float16.

    Same contract as cu_mlp_gemma2_fused_upproj_f32_v1 / _v2 (srcs/kernels/cuda/mlp_gemma2_fused_upproj.cuh:6-16).
    """
    _check_device(xt, wt_gp, wt_up)
    _require(wt_gp.dim() == 2 and tuple(wt_gp.shape) == tuple(wt_up.shape), "gate and up weights must agree")
    k, n = wt_gp.shape if b_layout == capi.B_ROW_MAJOR else (wt_gp.shape[1], wt_gp.shape[0])
    _require(xt.dim() >= 1 and xt.shape[-1] == k, "hidden size should match for xt and the weights")
    _require(xt.dtype in (torch.float32, torch.float16) and all(t.dtype == xt.dtype for t in (wt_gp, wt_up)), "Unsupported data types")
    _require(xt.is_contiguous() and wt_gp.is_contiguous() and wt_up.is_contiguous(), "dense operands expected")
    m = xt.numel() // k if k else 0
    out = torch.empty(tuple(xt.shape[:-1]) + (n,), dtype=xt.dtype, device=xt.device)
    fn_name = "anygpu_gemm_f16_f32acc_gelu_mul" if xt.dtype == torch.float16 else "anygpu_gemm_f32_gelu_mul"
    rc = getattr(capi.load(), fn_name)(xt.data_ptr(), wt_gp.data_ptr(), wt_up.data_ptr(), out.data_ptr(),
                                       m, n, k, max(k, 1), max(wt_gp.shape[1], 1), max(n, 1), b_layout, _stream_ptr())
    capi.check(fn_name, rc)
    return out


def tensor_softmax(x: torch.Tensor, out: torch.Tensor | None = None, *, alpha: float = 1.0, softcap: float = 0.0,
                   causal: bool = False, window: int = 0, q_len: int = 0, diag: int = 0) -> torch.Tensor:
    """Row softmax of a 2-D tensor with the fused prologue (scale -> softcap -> masks)."""
    _check_device(x)
    _require(x.dim() == 2, "softmax expects 2 dimensional tensors")
    _require(x.stride(1) == 1 or x.shape[1] <= 1, "rows must be contiguous")
    rows, cols = x.shape
    if out is None:
        out = torch.empty((rows, cols), dtype=x.dtype, device=x.device)
    _require(tuple(out.shape) == (rows, cols), "result shape is wrong")
    xs = x.stride(0) if rows > 1 else max(cols, 1)
    ys = out.stride(0) if rows > 1 else max(cols, 1)
    lib = capi.load()
    if x.dtype == torch.float16:
        fn, name = lib.anygpu_softmax_rows_f16, "anygpu_softmax_rows_f16"
    elif x.dtype == torch.float32:
        fn, name = lib.anygpu_softmax_rows_f32, "anygpu_softmax_rows_f32"
    else:
        raise TypeError("Unsupported data type")
    rc = fn(x.data_ptr(), out.data_ptr(), rows, cols, xs, ys, q_len, diag, alpha, softcap, int(causal), window,
            _stream_ptr())
    capi.check(name, rc)
    return out


def tensor_causal_conv1d(xt: torch.Tensor, wt: torch.Tensor, bt: torch.Tensor,
                         out: torch.Tensor | None = None) -> torch.Tensor:
    """silu(depthwise causal conv1d(xt, wt) + bt); xt [batch, dims, seq_len], wt [dims, width], bt [dims]."""
    _check_device(xt, wt, bt)
    _require(xt.dim() == 3, "xt needs to be 3 dimensional")
    _require(xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims")
    _require(wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims")
    _require(wt.shape[1] <= 4, "kernel width needs to be under 4")
    _require(xt.dtype == wt.dtype == bt.dtype, "operands must share a dtype")
    _require(xt.is_contiguous() and wt.is_contiguous() and bt.is_contiguous(), "dense operands expected")
    if out is None:
        out = torch.empty_like(xt)
    b, d, s = xt.shape
    lib = capi.load()
    if xt.dtype == torch.float16:
        fn, name = lib.anygpu_causal_conv1d_silu_f16, "anygpu_causal_conv1d_silu_f16"
    elif xt.dtype == torch.float32:
        fn, name = lib.anygpu_causal_conv1d_silu_f32, "anygpu_causal_conv1d_silu_f32"
    else:
        raise TypeError("Unsupported data types")
    rc = fn(xt.data_ptr(), wt.data_ptr(), bt.data_ptr(), out.data_ptr(), b, d, s, wt.shape[1], _stream_ptr())
    capi.check(name, rc)
    return out


def tensor_causal_conv1d_update(xt: torch.Tensor, state: torch.Tensor, wt: torch.Tensor, bt: torch.Tensor) -> torch.Tensor:
    """One decode step of tensor_causal_conv1d: xt [batch, dims] is the new sample of every row, state
    [batch, dims, width - 1] holds the samples in front of it (oldest first) and is updated in place."""
    _check_device(xt, state, wt, bt)
    _require(xt.dim() == 2 and state.dim() == 3, "xt needs to be 2 and state 3 dimensional")
    _require(xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims")
    _require(wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims")
    _require(wt.shape[1] <= 4, "kernel width needs to be under 4")
    _require(tuple(state.shape) == (xt.shape[0], xt.shape[1], wt.shape[1] - 1), "state needs to be (batch, dims, width - 1)")
    _require(xt.dtype == wt.dtype == bt.dtype == state.dtype, "operands must share a dtype")
    _require(all(t.is_contiguous() for t in (xt, state, wt, bt)), "dense operands expected")
    out = torch.empty_like(xt)
    lib = capi.load()
    if xt.dtype == torch.float16:
        fn, name = lib.anygpu_causal_conv1d_silu_update_f16, "anygpu_causal_conv1d_silu_update_f16"
    elif xt.dtype == torch.float32:
        fn, name = lib.anygpu_causal_conv1d_silu_update_f32, "anygpu_causal_conv1d_silu_update_f32"
    else:
        raise TypeError("Unsupported data types")
    rc = fn(xt.data_ptr(), state.data_ptr() if state.numel() else None, wt.data_ptr(), bt.data_ptr(), out.data_ptr(),
            xt.shape[0], xt.shape[1], wt.shape[1], _stream_ptr())
    capi.check(name, rc)
    return out


def tensor_rms_norm(xt: torch.Tensor, wt: torch.Tensor, eps: float, zero_centered: bool = False,
                    gate: torch.Tensor | None = None) -> torch.Tensor:
    """rms_norm(xt * silu(gate)) * (wt + zero_centered) over the last axis; gate None: plain RMS norm."""
    _check_device(xt, wt) if gate is None else _check_device(xt, wt, gate)
    _require(wt.dim() == 1 and xt.dim() >= 1 and xt.shape[-1] == wt.shape[0], "wt shape is incorrect")
    _require(gate is None or tuple(gate.shape) == tuple(xt.shape), "tensors are not elementwise compatible")
    _require(xt.dtype == wt.dtype and (gate is None or gate.dtype == xt.dtype), "operands must share a dtype")
    _require(xt.is_contiguous() and wt.is_contiguous() and (gate is None or gate.is_contiguous()), "dense operands expected")
    cols = wt.shape[0]
    rows = xt.numel() // cols if cols else 0
    out = torch.empty_like(xt)
    lib = capi.load()
    if xt.dtype == torch.float16:
        fn, name = lib.anygpu_gated_rmsnorm_f16, "anygpu_gated_rmsnorm_f16"
    elif xt.dtype == torch.float32:
        fn, name = lib.anygpu_gated_rmsnorm_f32, "anygpu_gated_rmsnorm_f32"
    else:
        raise TypeError("Unsupported data types")
    rc = fn(xt.data_ptr(), None if gate is None else gate.data_ptr(), wt.data_ptr(), out.data_ptr(), rows, cols,
            float(eps), int(zero_centered), _stream_ptr())
    capi.check(name, rc)
    return out


def tensor_zamba_gated_rmsnorm(xt: torch.Tensor, zt: torch.Tensor, wt: torch.Tensor, gsize: int, eps: float) -> torch.Tensor:
    """Same contract as tensor_zamba_gated_rmsnorm of the reference (srcs/models/zamba2/zamba_gated_rmsnorm.hpp:9-23):
    one group spans the row, gsize is accepted and, as there, not used."""
    return tensor_rms_norm(xt, wt, eps, False, gate=zt)


def tensor_mm_batched(lhs: torch.Tensor, rhs: torch.Tensor, b_layout: int = capi.B_ROW_MAJOR) -> torch.Tensor:
    """out[i] = lhs[i] @ B[i] for dense 3-D operands [batch, M, K] and [batch, K, N] (or [batch, N, K] with
    B_COL_MAJOR) in one launch: the per-head loop of the reference's attention collapsed."""
    _check_device(lhs, rhs)
    _require(lhs.dim() == 3 and rhs.dim() == 3 and lhs.shape[0] == rhs.shape[0], "batched operands must be 3-D")
    _require(lhs.dtype == rhs.dtype and lhs.is_contiguous() and rhs.is_contiguous(), "dense operands of one dtype expected")
    batch, m, k = lhs.shape
    n = rhs.shape[2] if b_layout == capi.B_ROW_MAJOR else rhs.shape[1]
    _require((rhs.shape[1] if b_layout == capi.B_ROW_MAJOR else rhs.shape[2]) == k,
             "matrix multiplication requires compatible matrices")
    out = torch.empty((batch, m, n), dtype=lhs.dtype, device=lhs.device)
    lib = capi.load()
    lda, ldb, ldc = max(k, 1), max(rhs.shape[2], 1), max(n, 1)
    if lhs.dtype == torch.float16:
        rc = lib.anygpu_gemm_f16_f32acc_batched(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), m, n, k, lda, ldb, ldc,
                                                m * k, n * k, m * n, batch, b_layout, _stream_ptr())
        capi.check("anygpu_gemm_f16_f32acc_batched", rc)
    elif lhs.dtype == torch.float32:
        rc = lib.anygpu_gemm_f32_batched(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), m, n, k, lda, ldb, ldc,
                                         m * k, n * k, m * n, batch, capi.A_ROW_MAJOR, b_layout, _stream_ptr())
        capi.check("anygpu_gemm_f32_batched", rc)
    else:
        raise TypeError("Unsupported data type")
    return out


def tensor_softmax_masked(x: torch.Tensor, mask: torch.Tensor, *, alpha: float = 1.0, softcap: float = 0.0,
                          q_len: int = 0) -> torch.Tensor:
    """softmax(softcap(alpha * x) + mask[r % q_len]) over the rows of a dense 2-D tensor; mask is a dense
    additive [q_len, cols] matrix of the same dtype."""
    _check_device(x, mask)
    _require(x.dim() == 2 and mask.dim() == 2 and mask.shape[1] == x.shape[1], "mask shape does not fit the scores")
    _require(x.dtype == mask.dtype and x.is_contiguous() and mask.is_contiguous(), "dense operands of one dtype expected")
    rows, cols = x.shape
    out = torch.empty_like(x)
    lib = capi.load()
    if x.dtype == torch.float16:
        fn, name = lib.anygpu_softmax_rows_masked_f16, "anygpu_softmax_rows_masked_f16"
    elif x.dtype == torch.float32:
        fn, name = lib.anygpu_softmax_rows_masked_f32, "anygpu_softmax_rows_masked_f32"
    else:
        raise TypeError("Unsupported data type")
    pitch = max(cols, 1)
    rc = fn(x.data_ptr(), mask.data_ptr(), out.data_ptr(), rows, cols, pitch, pitch, pitch, q_len, alpha, softcap,
            _stream_ptr())
    capi.check(name, rc)
    return out


def sdp_attention_masked_scaled_fwd(qw: torch.Tensor, kw: torch.Tensor, vw: torch.Tensor, mask: torch.Tensor,
                                    alpha: float) -> torch.Tensor:
    """softmax(alpha q k^T + mask) v over [..., n, d] tensors (reference: srcs/transformers/sdp.hpp:207-274):
    one batched GEMM for q k^T (k in its own storage), one fused softmax, one batched GEMM for p v."""
    _require(qw.dim() == kw.dim() == vw.dim() == mask.dim() and qw.dim() >= 2, "dimension missmatch")
    n_q, d = qw.shape[-2:]
    n_k, d_v = kw.shape[-2], vw.shape[-1]
    lead = qw.shape[:-2]
    _require(all(s == 1 for s in mask.shape[:-2]), "mask needs to have 1s in the first dims except the last two")
    if (qw.dtype in (torch.float32, torch.float16) and kw.dtype == vw.dtype == mask.dtype == qw.dtype and d == d_v and d in (64, 128, 256)
            and kw.shape[:-2] == qw.shape[:-2] and n_q > 0 and qw.numel() > 0 and n_k > 0):
        # one kernel that reads the mask as data, no score matrix in memory
        _check_device(qw, kw, vw, mask)
        q4, k4, v4, m2 = qw.contiguous(), kw.contiguous(), vw.contiguous(), mask.reshape(n_q, n_k).contiguous()
        out = torch.empty_like(q4)
        name = "anygpu_sdp_attention_fwd_masked_f32" if qw.dtype == torch.float32 else "anygpu_sdp_attention_fwd_masked_f16"
        rc = getattr(capi.load(), name)(q4.data_ptr(), k4.data_ptr(), v4.data_ptr(), m2.data_ptr(), out.data_ptr(),
                                        q4.numel() // (n_q * d), 1, n_q, n_k, d, n_k, float(alpha), 0.0, _stream_ptr())
        capi.check(name, rc)
        return out
    q3, k3, v3 = qw.reshape(-1, n_q, d), kw.reshape(-1, n_k, d), vw.reshape(-1, n_k, d_v)
    scores = tensor_mm_batched(q3.contiguous(), k3.contiguous(), b_layout=capi.B_COL_MAJOR)
    probs = tensor_softmax_masked(scores.reshape(-1, n_k), mask.reshape(n_q, n_k).contiguous(), alpha=alpha, q_len=n_q)
    out = tensor_mm_batched(probs.reshape(-1, n_q, n_k), v3.contiguous())
    return out.reshape(*lead, n_q, d_v)


def sdp_attention_fwd(qw: torch.Tensor, kw: torch.Tensor, vw: torch.Tensor, alpha: float, *, softcap: float = 0.0,
                      causal: bool = False, window: int = 0, decode: bool | None = None) -> torch.Tensor:
    """softmax(mask(softcap(alpha q k^T))) v in one kernel; q [..., heads, n_q, d], k and v [..., kv_heads, n_k, d]
    with heads a multiple of kv_heads, float16 or float32; masks are index rules with the causal diagonal at
    n_k - n_q.  decode: True / False forces the split-key decode form or the fused form, None picks by shape."""
    _check_device(qw, kw, vw)
    _require(qw.dim() == kw.dim() == vw.dim() and qw.dim() >= 3, "dimension missmatch")
    _require(qw.dtype == kw.dtype == vw.dtype and qw.dtype in (torch.float16, torch.float32), "Unsupported data types")
    _require(tuple(kw.shape) == tuple(vw.shape) and kw.shape[-1] == qw.shape[-1], "q, k and v need one head dimension")
    _require(qw.shape[:-3] == kw.shape[:-3] and kw.shape[-3] > 0 and qw.shape[-3] % kw.shape[-3] == 0,
             "query heads need to be a multiple of key / value heads")
    _require(qw.is_contiguous() and kw.is_contiguous() and vw.is_contiguous(), "dense operands expected")
    heads, n_q, d = qw.shape[-3:]
    kv_heads, n_k = kw.shape[-3], kw.shape[-2]
    batch_heads = qw.numel() // (n_q * d) if n_q * d else 0
    q_per_kv = heads // kv_heads
    out = torch.empty_like(qw)
    lib = capi.load()
    if decode is None:
        # generation steps: few rows per key / value head and enough keys for the split to pay; up to 128 rows of up to
        # 16 queries per head where the fused form (a block per head and 128 queries) would leave half of the chip idle
        rows = q_per_kv * n_q
        decode = n_k >= 256 and d in (64, 128, 256) and (0 < rows <= 16 or (rows <= 128 and n_q <= 16 and batch_heads <= 128))
    if qw.dtype == torch.float32:
        if decode:
            need = lib.anygpu_sdp_attention_decode_f32_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, d, int(causal), int(window))
            capi.check("anygpu_sdp_attention_decode_f32_workspace_bytes", min(int(need), 0))
            workspace = torch.empty(max(int(need), 16), dtype=torch.uint8, device=qw.device)
            rc = lib.anygpu_sdp_attention_decode_f32(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), out.data_ptr(),
                                                     workspace.data_ptr(), workspace.numel(), batch_heads, q_per_kv, n_q, n_k, d,
                                                     float(alpha), float(softcap), int(causal), int(window), _stream_ptr())
            capi.check("anygpu_sdp_attention_decode_f32", rc)
            return out
        rc = lib.anygpu_sdp_attention_fwd_f32(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), out.data_ptr(),
                                              batch_heads, q_per_kv, n_q, n_k, d, float(alpha),
                                              float(softcap), int(causal), int(window), _stream_ptr())
        capi.check("anygpu_sdp_attention_fwd_f32", rc)
        return out
    if decode:
        need = lib.anygpu_sdp_attention_decode_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, d, int(causal), int(window))
        capi.check("anygpu_sdp_attention_decode_workspace_bytes", min(int(need), 0))
        workspace = torch.empty(max(int(need), 16), dtype=torch.uint8, device=qw.device)
        rc = lib.anygpu_sdp_attention_decode_f16(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), out.data_ptr(),
                                                 workspace.data_ptr(), workspace.numel(), batch_heads, q_per_kv, n_q, n_k, d,
                                                 float(alpha), float(softcap), int(causal), int(window), _stream_ptr())
        capi.check("anygpu_sdp_attention_decode_f16", rc)
        return out
    rc = lib.anygpu_sdp_attention_fwd_f16(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), out.data_ptr(),
                                          batch_heads, q_per_kv, n_q, n_k, d, float(alpha),
                                          float(softcap), int(causal), int(window), _stream_ptr())
    capi.check("anygpu_sdp_attention_fwd_f16", rc)
    return out
