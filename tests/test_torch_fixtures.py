"""Parity against expected values that do NOT come from the CPU oracle: the fixtures under
tests/golden/torch_* were written by tests/golden/make_torch_fixtures.py from PyTorch's library
routines in float64 (the one-line formulas the reference's own generators use).  The CPU tests
hold the oracle to them, the GPU tests hold the HIP kernels (through the C ABI) to them, each
at the tolerance stated for the operator.
"""
import math
import sys
from pathlib import Path

import numpy as np
import pytest

from helpers import scaled_rel_err

GOLDEN = Path(__file__).resolve().parent / "golden"
sys.path.insert(0, str(GOLDEN))

from dat_codec import load_tensor  # noqa: E402

TOL_F16_GEMM = 1e-2      # fp16 inputs, fp32 accumulation, fp16 output
TOL_F32 = 1e-4           # float32 operators
TOL_F16_ROWOPS = 2e-3    # fp16 softmax / conv1d; attention on fp16 inputs passes through two products: 2 x this


def case(name, *files):
    d = GOLDEN / name
    return tuple(load_tensor(d / f"{f}.dat") for f in files)


def up(a):
    return a.astype(np.float32)


# ---------------------------------------------------------------------------------------------
# the oracle against torch (CPU)
# ---------------------------------------------------------------------------------------------

def test_oracle_mm_vs_torch_matmul(oracle):
    x, w, y = case("torch_mm_m24_n16_k40_f32", "x", "w", "y")
    assert scaled_rel_err(oracle.tensor_mm(x, w), y, math.sqrt(40) / 3) <= 1e-6
    x, w, y = case("torch_mm_m64_n64_k128_f16", "x", "w", "y")
    assert scaled_rel_err(oracle.tensor_mm(oracle.cvt_f16_to_f32(x), oracle.cvt_f16_to_f32(w)), y, math.sqrt(128) / 3) <= 1e-6


def test_oracle_sdp_masked_scaled_vs_torch_sdpa(oracle):
    q, k, v, mask, y = case("torch_sdp_fwd_masked_scaled_f32", "q", "k", "v", "mask", "y")
    assert np.max(np.abs(oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask, 0.125) - y)) <= 1e-5
    # the same case through the rule form (causal rule = the tril -inf mask)
    assert np.max(np.abs(oracle.sdp_attention_rules(q[0], k[0], v[0], alpha=0.125, causal=True) - y[0])) <= 1e-5


def test_oracle_sdp_rules_gqa_vs_torch(oracle):
    q, k, v, y = case("torch_sdp_gqa_window_f16", "q", "k", "v", "y")
    got = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t)[0] for t in (q, k, v)), alpha=0.125, causal=True,
                                     window=9, q_per_kv=3)
    assert np.max(np.abs(got - y[0])) <= 1e-5
    q, k, v, y = case("torch_sdp_gqa_softcap_window_f32_d256", "q", "k", "v", "y")
    got = oracle.sdp_attention_rules(q[0], k[0], v[0], alpha=0.0625, softcap=50.0, causal=True, window=10, q_per_kv=2)
    assert np.max(np.abs(got - y[0])) <= 1e-5


def test_oracle_softmax_vs_torch(oracle):
    x, y, vis = case("torch_softmax_softcap_window_f32", "scores", "y", "visible")
    got = oracle.attention_softmax(x, alpha=0.0625, softcap=50.0, causal=True, window=6, q_len=16)
    assert np.max(np.abs(got - y)) <= 1e-6
    assert np.all(got[vis == 0] == 0.0) and np.all(y[vis == 0] == 0.0)
    x, y = case("torch_softmax_causal_scaled_f32", "scores", "y")
    assert np.max(np.abs(oracle.attention_softmax(x, alpha=0.125, causal=True, q_len=24) - y)) <= 1e-6


def test_oracle_conv1d_vs_torch(oracle):
    for name in ("torch_causal_conv1d_fwd_f32", "torch_causal_conv1d_fwd_w3_f32"):
        x, w, b, y = case(name, "x", "w", "b", "y")
        assert np.max(np.abs(oracle.tensor_causal_conv1d(x, w, b) - y)) <= 2e-6


def test_oracle_conv1d_update_vs_torch(oracle):
    for name in ("torch_causal_conv1d_update_f32", "torch_causal_conv1d_update_w2_f32"):
        state, x, w, b, y, new_state = case(name, "state", "x", "w", "b", "y", "new_state")
        got, got_state = oracle.causal_conv1d_update(x, state, w, b)
        assert np.max(np.abs(got - y)) <= 2e-6
        assert np.array_equal(got_state, new_state)


def test_oracle_gated_rmsnorm_vs_torch(oracle):
    x, z, w, y = case("torch_gated_rmsnorm_f32", "in_0", "in_1", "weight", "out_0")
    assert np.max(np.abs(oracle.zamba_gated_rmsnorm(x, z, w, 1e-5) - y)) <= 1e-5


def test_oracle_gemma2_epilogues_vs_torch(oracle):
    x, w, y = case("torch_gemma2_lmhead_softcap_f32", "x", "w", "y")
    assert np.max(np.abs(oracle.gemma_linear_softcap(x[None], w, 30.0)[0] - y)) <= 2e-5
    x, wg, wu, y = case("torch_gemma2_mlp_upproj_f32", "x", "w_gate", "w_up", "y")
    got = oracle.gemma_mlp_upproj(x[None], np.ascontiguousarray(wg.T), np.ascontiguousarray(wu.T))[0]
    assert np.max(np.abs(got - y)) <= 1e-5


# ---------------------------------------------------------------------------------------------
# the HIP kernels against torch (GPU, through the C ABI)
# ---------------------------------------------------------------------------------------------

def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


@pytest.mark.gpu
def test_hip_mm_vs_torch_matmul(ops):
    x, w, y = case("torch_mm_m24_n16_k40_f32", "x", "w", "y")
    assert scaled_rel_err(host(ops.tensor_mm(dev(x), dev(w))), y, math.sqrt(40) / 3) <= TOL_F32
    x, w, y = case("torch_mm_m64_n64_k128_f16", "x", "w", "y")
    assert scaled_rel_err(up(host(ops.tensor_mm(dev(x), dev(w)))), y, math.sqrt(128) / 3) <= TOL_F16_GEMM


@pytest.mark.gpu
def test_hip_sdp_vs_torch_sdpa(ops):
    q, k, v, mask, y = case("torch_sdp_fwd_masked_scaled_f32", "q", "k", "v", "mask", "y")
    # the three-launch form with the mask handed over as data, and the fused kernel with the causal rule
    got = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask), 0.125))
    assert scaled_rel_err(got, y, 1.0) <= TOL_F32
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.125, causal=True))
    assert scaled_rel_err(got, y, 1.0) <= TOL_F32


@pytest.mark.gpu
def test_hip_sdp_gqa_vs_torch(ops):
    q, k, v, y = case("torch_sdp_gqa_window_f16", "q", "k", "v", "y")
    got = up(host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.125, causal=True, window=9)))
    assert scaled_rel_err(got, y, 1.0) <= 2 * TOL_F16_ROWOPS
    q, k, v, y = case("torch_sdp_gqa_softcap_window_f32_d256", "q", "k", "v", "y")
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0625, softcap=50.0, causal=True, window=10))
    assert scaled_rel_err(got, y, 1.0) <= TOL_F32
    # the same case in half precision through the fp16 kernel of head dimension 256
    got = up(host(ops.sdp_attention_fwd(dev(q.astype(np.float16)), dev(k.astype(np.float16)), dev(v.astype(np.float16)),
                                        0.0625, softcap=50.0, causal=True, window=10)))
    assert scaled_rel_err(got, y, 1.0) <= 1e-2     # inputs themselves rounded to half here: the fp16 GEMM tolerance


@pytest.mark.gpu
def test_hip_softmax_vs_torch(ops):
    x, y, vis = case("torch_softmax_softcap_window_f32", "scores", "y", "visible")
    kw = dict(alpha=0.0625, softcap=50.0, causal=True, window=6, q_len=16)
    got = host(ops.tensor_softmax(dev(x), **kw))
    assert scaled_rel_err(got, y, y.max(axis=1, keepdims=True)) <= TOL_F32
    assert np.all(got[vis == 0] == 0.0)
    xh = x.astype(np.float16)
    got = up(host(ops.tensor_softmax(dev(xh), **kw)))
    import torch
    z = 50.0 * torch.tanh(torch.from_numpy(xh).double() * 0.0625 / 50.0)
    yh = torch.softmax(torch.where(torch.from_numpy(vis) != 0, z, torch.tensor(float("-inf"), dtype=torch.float64)), -1).numpy()
    assert scaled_rel_err(got, yh, yh.max(axis=1, keepdims=True)) <= TOL_F16_ROWOPS
    assert np.all(got[vis == 0] == 0.0)
    x, y = case("torch_softmax_causal_scaled_f32", "scores", "y")
    got = host(ops.tensor_softmax(dev(x), alpha=0.125, causal=True, q_len=24))
    assert scaled_rel_err(got, y, y.max(axis=1, keepdims=True)) <= TOL_F32


@pytest.mark.gpu
def test_hip_conv1d_vs_torch(ops):
    for name in ("torch_causal_conv1d_fwd_f32", "torch_causal_conv1d_fwd_w3_f32"):
        x, w, b, y = case(name, "x", "w", "b", "y")
        assert scaled_rel_err(host(ops.tensor_causal_conv1d(dev(x), dev(w), dev(b))), y, 1.0) <= TOL_F32
    # half precision: the same torch formula on the half-rounded inputs
    import torch
    import torch.nn.functional as F
    x, w, b, _ = case("torch_causal_conv1d_fwd_f32", "x", "w", "b", "y")
    xh, wh, bh = (t.astype(np.float16) for t in (x, w, b))
    tx, tw, tb = (torch.from_numpy(t).double() for t in (xh, wh, bh))
    yh = F.silu(F.conv1d(tx, tw.unsqueeze(1), tb, padding=w.shape[1] - 1, groups=w.shape[0]))[..., :x.shape[2]].numpy()
    assert scaled_rel_err(up(host(ops.tensor_causal_conv1d(dev(xh), dev(wh), dev(bh)))), yh, 1.0) <= TOL_F16_ROWOPS


@pytest.mark.gpu
def test_hip_conv1d_update_vs_torch(ops):
    for name in ("torch_causal_conv1d_update_f32", "torch_causal_conv1d_update_w2_f32"):
        state, x, w, b, y, new_state = case(name, "state", "x", "w", "b", "y", "new_state")
        dstate = dev(state)
        got = host(ops.tensor_causal_conv1d_update(dev(x), dstate, dev(w), dev(b)))
        assert scaled_rel_err(got, y, 1.0) <= TOL_F32
        assert np.array_equal(host(dstate), new_state)


@pytest.mark.gpu
def test_hip_gated_rmsnorm_vs_torch(ops):
    x, z, w, y = case("torch_gated_rmsnorm_f32", "in_0", "in_1", "weight", "out_0")
    got = host(ops.tensor_zamba_gated_rmsnorm(dev(x), dev(z), dev(w), 96, 1e-5))
    assert scaled_rel_err(got, y, 1.0) <= TOL_F32


@pytest.mark.gpu
def test_hip_gemma2_epilogues_vs_torch(ops):
    x, w, y = case("torch_gemma2_lmhead_softcap_f32", "x", "w", "y")
    got = host(ops.tensor_gemma_linear_softcap(dev(x[None]), dev(w), 30.0))[0]
    assert scaled_rel_err(got, y, 30.0) <= TOL_F32
    x, wg, wu, y = case("torch_gemma2_mlp_upproj_f32", "x", "w_gate", "w_up", "y")
    got = host(ops.mlp_gemma2_fused_upproj(dev(x[None]), dev(np.ascontiguousarray(wg.T)), dev(np.ascontiguousarray(wu.T))))[0]
    assert scaled_rel_err(got, y, 1.0) <= TOL_F32
