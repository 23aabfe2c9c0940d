"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on identical
inputs.  Tolerances (scale-floored relative error, see tests/helpers.py):
    fp16-in / fp32-accumulate GEMM  <= 1e-2      fp32 ops  <= 1e-4      fp16 softmax / conv1d  <= 2e-3
Integer-valued cases are bit exact.  Masked softmax outputs must be exactly 0.
"""
import ctypes
import math

import numpy as np
import pytest

from anygpu_amd import synth
from helpers import exact_int_product, rel_l2, sample_rows, scaled_rel_err

pytestmark = pytest.mark.gpu

TOL_F16_GEMM = 1e-2
TOL_F32 = 1e-4
TOL_F16_ROWOPS = 2e-3



def mm_want(oracle, a, b, macs=1.0e8):
    """a @ b as the parity checks of the larger products take it.  Up to `macs` multiply-adds the oracle computes the
    whole product the reference's way.  Beyond that (the reference's loop order takes minutes there) the whole product
    comes from float64 BLAS, exact for the integer-valued operands of the bit-exact tests and closer to the true sums
    than any float32 summation otherwise, and the oracle's own values are written over a sample of rows (first, last
    and a seeded spread) and, where the rows are few, of columns; for integer-valued operands the two have to agree
    bit for bit on the sample."""
    m, k = a.shape
    n = b.shape[1]
    if float(m) * k * n <= macs:
        return oracle.tensor_mm(a, b, threads=8)
    full = (a.astype(np.float64) @ b.astype(np.float64)).astype(a.dtype)
    rows = sample_rows(m, int(max(8, min(m, macs / (float(k) * n)))))
    cols = np.arange(n) if float(len(rows)) * k * n <= macs else sample_rows(n, int(max(64, macs / (float(len(rows)) * k))), seed=1)
    sub = oracle.tensor_mm(np.ascontiguousarray(a[rows]), np.ascontiguousarray(b[:, cols]), threads=8)
    if np.array_equal(a, np.rint(a)) and np.array_equal(b, np.rint(b)):
        assert np.array_equal(sub, full[np.ix_(rows, cols)])
    full[np.ix_(rows, cols)] = sub
    return full


def _rows_want(oracle_fn, blas_fn, x, macs_per_row, macs=1.0e8):
    """A row-wise operator over x [..., rows, k] for the parity checks of the larger shapes: the oracle computes all rows
    where that is up to `macs` multiply-adds; beyond, the whole result comes from blas_fn (products in float64 BLAS, the
    element-wise steps by the oracle's own functions) and the oracle's values the reference's way are written over a sample
    of rows (first, last and a seeded spread, at least 8)."""
    m = x.shape[-2]
    if float(m) * macs_per_row <= macs:
        return oracle_fn(x)
    full = blas_fn(x)
    rows = sample_rows(m, int(max(8, macs / macs_per_row)))
    full[..., rows, :] = oracle_fn(np.ascontiguousarray(x[..., rows, :]))
    return full


def _blas_mm(x, w):
    return (x.astype(np.float64) @ w.astype(np.float64)).astype(np.float32)


def gemm_want(oracle, a, b, bias):
    return _rows_want(lambda r: oracle.tensor_gemm(r, b, bias, threads=8), lambda r: oracle.tensor_add(_blas_mm(r, b), np.broadcast_to(bias, (r.shape[0], b.shape[1])).copy()),
                      a, float(b.shape[0]) * b.shape[1])


def softcap_head_want(oracle, x, w, cap):
    return _rows_want(lambda r: oracle.gemma_linear_softcap(r, w, cap, threads=8), lambda r: oracle.softcap(_blas_mm(r, w.T), cap).reshape(r.shape[:-1] + (w.shape[0],)),
                      x, float(w.shape[0]) * w.shape[1])


def upproj_want(oracle, x, wg, wu):
    return _rows_want(lambda r: oracle.gemma_mlp_upproj(r, wg, wu, threads=8),
                      lambda r: oracle.tensor_mul(oracle.tensor_gelu_tanh(_blas_mm(r, wg)), _blas_mm(r, wu)).reshape(r.shape[:-1] + (wg.shape[1],)),
                      x, 2.0 * wg.shape[0] * wg.shape[1])


def hide_key_stripes(mask, rng):
    """Hides long key ranges from long query ranges of an additive mask [n_q, n_k] in place (whole key tiles hidden from
    whole blocks of queries, their edges anywhere), the first keys among them; every query keeps one visible key, each
    somewhere else."""
    n_q, n_k = mask.shape
    for _ in range(6):
        r0, c0 = int(rng.integers(0, n_q)), int(rng.integers(0, n_k))
        mask[r0:r0 + int(rng.integers(40, 400)), c0:c0 + int(rng.integers(100, 1200))] = -np.inf
    mask[: n_q // 2, :200] = -np.inf
    mask[n_q // 3:, n_k - 300:] = -np.inf
    mask[np.arange(n_q), rng.integers(0, n_k, n_q)] = 0.25


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


# =============================================================================================
# softmax
# =============================================================================================

def test_softmax_f32_reference_case_6x45(ops, oracle):
    # tests/tests.cpp:187-204: crt_random_tensor (integers 0..10), CPU vs device, abs tol 1e-3
    x = synth.integers(11, (6, 45), 0, 10)
    got = host(ops.tensor_softmax(dev(x)))
    want = oracle.tensor_softmax(x)
    ok, worst = oracle.compare_data_buffers(got, want)
    assert ok, worst
    assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= TOL_F32


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 7), (5, 8), (64, 512), (33, 520), (17, 1024), (9, 2048),
                                       (6, 4096), (5, 8192), (3, 8200), (2, 16384), (4, 100), (7, 2047),
                                       (2, 20000), (3, 20001), (2, 32768), (1, 40000), (2, 33001),
                                       # many short rows (a row of 16 lanes each) and rows a block walks twice
                                       (200, 64), (77, 128), (100, 256), (65, 8), (130, 100), (300, 333), (1000, 500),
                                       (70, 50257), (3, 131072), (2, 262147), (300, 16400)])
def test_softmax_plain_shapes(ops, oracle, dtype, rows, cols):
    np_dt = np.float16 if dtype == "f16" else np.float32
    x = synth.normal(rows * 131 + cols, (rows, cols), std=2.0).astype(np_dt)
    got = host(ops.tensor_softmax(dev(x))).astype(np.float32)
    want = oracle.tensor_softmax(oracle.cvt_f16_to_f32(x) if dtype == "f16" else x)
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= tol
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < (2e-2 if dtype == "f16" else 1e-5))


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("rows,cols,causal,window,cap", [(5, 45, False, 0, 0.0), (64, 2047, True, 0, 0.0), (33, 1001, True, 300, 30.0),
                                                        (16, 8191, True, 0, 0.0), (9, 7, True, 3, 0.0), (12, 1337, False, 0, 20.0)])
def test_softmax_rows_at_element_alignment(ops, oracle, dtype, rows, cols, causal, window, cap):
    # widths that are no multiple of the 16-byte vector: rows start at element alignment, the last vector is partial
    import torch
    np_dt = np.float16 if dtype == "f16" else np.float32
    x = (synth.normal(rows + cols, (rows, cols)) * np.float32(3.0)).astype(np_dt)
    # the matrix sits in the middle of a flat buffer: the elements in front of and behind it must stay untouched
    flat_x = torch.full((rows * cols + 64,), 9.0, device="cuda", dtype=torch.float16 if dtype == "f16" else torch.float32)
    flat_y = torch.full_like(flat_x, -5.0)
    for front in (0, 1, 5):
        xv = flat_x[front:front + rows * cols].view(rows, cols)
        yv = flat_y[front:front + rows * cols].view(rows, cols)
        xv.copy_(dev(x))
        flat_y.fill_(-5.0)
        ops.tensor_softmax(xv, out=yv, alpha=0.5, softcap=cap, causal=causal, window=window, q_len=rows if causal else 0,
                           diag=cols - rows if causal else 0)
        got_flat = host(flat_y).astype(np.float32)
        got = got_flat[front:front + rows * cols].reshape(rows, cols)
        want = oracle.attention_softmax(oracle.cvt_f16_to_f32(x) if dtype == "f16" else x, alpha=0.5, softcap=cap, causal=causal,
                                        window=window, q_len=rows if causal else 0, diag=cols - rows if causal else 0)
        tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
        blind = np.isnan(want).all(axis=1)              # rows without a visible key: 0 / 0 in the operator chain, zeros here
        assert not got[blind].any()
        got, want = got[~blind], want[~blind]
        assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= tol
        assert np.all(got[want == 0.0] == 0.0)
        assert np.all(got_flat[:front] == -5.0) and np.all(got_flat[front + rows * cols:] == -5.0)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_softmax_padded_row_strides(ops, oracle, dtype):
    import torch
    np_dt = np.float16 if dtype == "f16" else np.float32
    rows, cols, pitch = 37, 256, 320
    buf = synth.normal(3, (rows, pitch), std=2.0).astype(np_dt)
    xb = dev(buf)
    out = torch.full((rows, pitch + 64), 7.0, dtype=xb.dtype, device="cuda")
    ops.tensor_softmax(xb[:, :cols], out=out[:, :cols])
    got = host(out).astype(np.float32)
    xin = buf[:, :cols]
    want = oracle.tensor_softmax(np.ascontiguousarray(oracle.cvt_f16_to_f32(xin) if dtype == "f16" else xin))
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    assert scaled_rel_err(got[:, :cols], want, want.max(axis=1, keepdims=True)) <= tol
    assert np.all(got[:, cols:] == 7.0)      # padding is not written


FUSED_CASES = [
    # rows, cols, q_len, diag, alpha, softcap, causal, window
    (64, 64, 64, 0, 0.125, 0.0, True, 0),
    (96, 48, 48, 0, 0.125, 0.0, True, 0),           # two heads of 48 queries
    (64, 64, 64, 0, 0.0625, 50.0, True, 16),
    (40, 72, 40, 32, 0.125, 0.0, True, 0),          # keys longer than queries: diagonal shifted
    (40, 72, 40, 32, 0.125, 30.0, True, 24),
    (33, 100, 33, 0, 1.0, 0.0, False, 10),          # window without causal, scalar kernel
    (128, 1024, 128, 896, 0.125, 0.0, True, 256),
    (50, 37, 25, 0, 0.3, 5.0, True, 7),
    (16, 8192, 16, 8176, 0.0625, 50.0, True, 4096),
    (8, 64, 8, -3, 0.125, 0.0, True, 0),            # first rows see nothing at all
    (128, 96, 64, 32, 0.25, 10.0, True, 20),        # many short rows, sixteen lanes per row
    (80, 200, 80, 120, 0.5, 0.0, True, 0),
    (4, 40000, 4, 39996, 0.1, 30.0, True, 1000),    # rows longer than a block's registers
    (3, 70001, 3, 69000, 0.05, 0.0, True, 0),
]


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("case", FUSED_CASES)
def test_softmax_fused_prologue(ops, oracle, dtype, case):
    rows, cols, q_len, diag, alpha, cap, causal, window = case
    np_dt = np.float16 if dtype == "f16" else np.float32
    x = synth.normal(rows + cols, (rows, cols), std=1.0 / alpha).astype(np_dt)
    got = host(ops.tensor_softmax(dev(x), alpha=alpha, softcap=cap, causal=causal, window=window,
                                  q_len=q_len, diag=diag)).astype(np.float32)
    x32 = oracle.cvt_f16_to_f32(x) if dtype == "f16" else x
    i = (np.arange(rows) % q_len)[:, None]
    j = np.arange(cols)[None, :]
    vis = np.ones((rows, cols), dtype=bool)
    if causal:
        vis &= j <= i + diag
    if window > 0:
        vis &= j > i + diag - window
    live = vis.any(axis=1)
    want = np.zeros((rows, cols), dtype=np.float32)
    if live.any():
        want[live] = oracle.attention_softmax(x32, alpha=alpha, softcap=cap, causal=causal, window=window,
                                              q_len=q_len, diag=diag, row_index=np.nonzero(live)[0])
    assert np.all(got[~vis] == 0.0), "masked outputs must be exact zeros"
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    floor = np.maximum(want.max(axis=1, keepdims=True), 1e-30)
    assert scaled_rel_err(got, want, floor) <= tol


def test_softmax_first_causal_row_and_neg_inf_inputs(ops):
    import torch
    x = torch.randn(4, 64, device="cuda", dtype=torch.float32)
    x[2, 5:] = float("-inf")
    x[3, :] = float("-inf")
    x[3, 9] = 0.5
    y = host(ops.tensor_softmax(x, causal=True, q_len=64, diag=60))
    # row 2 (query 2, sees keys 0..62): entries 5.. are -inf inputs -> exact zeros
    assert np.all(y[2, 5:] == 0.0) and abs(y[2, :5].sum() - 1.0) < 1e-6
    assert y[3, 9] == 1.0 and y[3].sum() == 1.0
    y0 = host(ops.tensor_softmax(x[:1], causal=True, q_len=64))
    assert y0[0, 0] == 1.0 and not y0[0, 1:].any()


def test_softmax_empty_and_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    e = ops.tensor_softmax(torch.empty((0, 16), device="cuda", dtype=torch.float16))
    assert e.shape == (0, 16)
    e = ops.tensor_softmax(torch.empty((4, 0), device="cuda", dtype=torch.float32))
    assert e.shape == (4, 0)
    x = torch.zeros((4, 16), device="cuda", dtype=torch.float32)
    y = torch.full((4, 16), 3.0, device="cuda", dtype=torch.float32)
    assert lib.anygpu_softmax_rows_f32(None, y.data_ptr(), 4, 16, 16, 16, 0, 0, 1.0, 0.0, 0, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert lib.anygpu_softmax_rows_f32(x.data_ptr(), y.data_ptr(), 4, 16, 8, 16, 0, 0, 1.0, 0.0, 0, 0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    assert lib.anygpu_softmax_rows_f32(x.data_ptr(), y.data_ptr(), -1, 16, 16, 16, 0, 0, 1.0, 0.0, 0, 0, None) == capi.ANYGPU_ERR_BAD_SHAPE
    assert lib.anygpu_softmax_rows_f32(x.data_ptr(), y.data_ptr(), 4, 16, 16, 16, 0, 0, 1.0, 0.0, 0, -2, None) == capi.ANYGPU_ERR_BAD_SHAPE
    torch.cuda.synchronize()
    assert bool((y == 3.0).all()), "a rejected call must not launch anything"


def _full_size_softmax(ops, oracle, heads, q, k, std, alpha, cap, window, n_sample):
    import torch
    rows = heads * q
    x = dev(synth.normal_matrix_f16(0, rows, k, std))          # the scores the benchmark times: seed 0, drawn on the host
    y = ops.tensor_softmax(x, alpha=alpha, softcap=cap, causal=True, window=window, q_len=q)
    torch.cuda.synchronize()
    # size-independent properties over the whole output
    sums = y.float().sum(dim=1)
    assert float((sums - 1.0).abs().max()) < 2e-2
    i = (torch.arange(rows, device="cuda") % q)[:, None]
    # masked region must be exactly zero: check in row slabs to bound memory
    for r0 in range(0, rows, 8192):
        blk = y[r0:r0 + 8192]
        ii = i[r0:r0 + 8192]
        j = torch.arange(k, device="cuda")[None, :]
        masked = j > ii
        if window > 0:
            masked |= j <= ii - window
        assert not bool(blk[masked].any())
    # sampled rows against the oracle on the very same fp16 inputs
    idx = sample_rows(rows, n_sample, seed=1)
    xs = x[torch.from_numpy(idx).cuda()].cpu().numpy()
    # a sampled row arrives alone, so its query index is handed to the oracle as the diagonal shift
    want = np.zeros((idx.size, k), dtype=np.float32)
    x32 = oracle.cvt_f16_to_f32(xs)
    for t, r in enumerate(idx):
        want[t] = oracle.attention_softmax(x32[t:t + 1], alpha=alpha, softcap=cap, causal=True, window=window,
                                           q_len=0, diag=int(r % q))[0]
    got = y[torch.from_numpy(idx).cuda()].cpu().numpy().astype(np.float32)
    assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= TOL_F16_ROWOPS


def test_softmax_config_causal_32x2048x2048(ops, oracle):
    _full_size_softmax(ops, oracle, heads=32, q=2048, k=2048, std=4.0, alpha=1.0 / 8.0, cap=0.0, window=0, n_sample=96)


def test_softmax_config_gemma2_8x8192x8192(ops, oracle):
    _full_size_softmax(ops, oracle, heads=8, q=8192, k=8192, std=16.0, alpha=1.0 / 16.0, cap=50.0, window=4096,
                       n_sample=48)


# =============================================================================================
# causal conv1d + SiLU
# =============================================================================================

def _conv_case(ops, oracle, dtype, b, d, s, width, seed, threads=8):
    np_dt = np.float16 if dtype == "f16" else np.float32
    x = synth.normal(seed, (b, d, s)).astype(np_dt)
    w = synth.normal(seed + 1, (d, width), std=0.5).astype(np_dt)
    bias = synth.normal(seed + 2, (d,), std=0.1).astype(np_dt)
    got = host(ops.tensor_causal_conv1d(dev(x), dev(w), dev(bias))).astype(np.float32)
    if dtype == "f16":
        x, w, bias = (oracle.cvt_f16_to_f32(v) for v in (x, w, bias))
    want = oracle.tensor_causal_conv1d(x, w, bias, threads=threads)
    return got, want


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("b,d,s,width", [(1, 1, 1, 1), (2, 3, 5, 4), (2, 5, 64, 4), (1, 7, 520, 3), (3, 4, 4096, 4),
                                         (2, 3, 8192, 2), (1, 2, 12296, 4), (2, 6, 638, 4), (1, 3, 2048, 1),
                                         (2, 2, 4104, 4), (1, 5, 33, 2)])
def test_conv1d_shapes(ops, oracle, dtype, b, d, s, width):
    got, want = _conv_case(ops, oracle, dtype, b, d, s, width, seed=b * 1000 + d * 100 + s)
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    assert scaled_rel_err(got, want, 1.0) <= tol


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("b,d,s,width", [(2, 5, 638, 4), (1, 3, 4095, 4), (3, 4, 9, 3), (2, 7, 17, 2), (1, 2, 1031, 4)])
def test_conv1d_rows_at_element_alignment(ops, oracle, dtype, b, d, s, width):
    # sequence lengths that are no multiple of the 16-byte vector; tensors in the middle of a flat buffer whose
    # surroundings must stay untouched
    import torch
    np_dt = np.float16 if dtype == "f16" else np.float32
    t_dt = torch.float16 if dtype == "f16" else torch.float32
    x = synth.normal(b * d + s, (b, d, s)).astype(np_dt)
    w = (synth.normal(1, (d, width)) * np.float32(0.5)).astype(np_dt)
    bias = (synth.normal(2, (d,)) * np.float32(0.1)).astype(np_dt)
    up = (lambda a: oracle.cvt_f16_to_f32(a)) if dtype == "f16" else (lambda a: a)
    want = oracle.tensor_causal_conv1d(up(x), up(w), up(bias))
    n = b * d * s
    flat_x = torch.full((n + 64,), 9.0, device="cuda", dtype=t_dt)
    flat_y = torch.full_like(flat_x, -5.0)
    for front in (0, 1, 6):
        xv = flat_x[front:front + n].view(b, d, s)
        yv = flat_y[front:front + n].view(b, d, s)
        xv.copy_(dev(x))
        flat_y.fill_(-5.0)
        ops.tensor_causal_conv1d(xv, dev(w), dev(bias), out=yv)
        got_flat = host(flat_y).astype(np.float32)
        got = got_flat[front:front + n].reshape(b, d, s)
        assert scaled_rel_err(got, want, 1.0) <= (TOL_F16_ROWOPS if dtype == "f16" else TOL_F32)
        assert np.all(got_flat[:front] == -5.0) and np.all(got_flat[front + n:] == -5.0)


def test_conv1d_f32_reference_generator_shape(ops, oracle):
    # tests/ext_torch_tests.cpp:745-778 (batch 8, dims 2318, seq 638, width 4), gate: abs tol 1e-3
    got, want = _conv_case(ops, oracle, "f32", 8, 2318, 638, 4, seed=10)
    ok, worst = oracle.compare_data_buffers(got, want)
    assert ok, worst
    assert scaled_rel_err(got, want, 1.0) <= TOL_F32


def test_conv1d_config_zamba2_4x4224x4096_f16(ops, oracle):
    import torch
    b, d, s, width = 4, 4224, 4096, 4
    x = synth.normal(0, (b, d, s)).astype(np.float16)
    w = synth.normal(1, (d, width), std=0.5).astype(np.float16)
    bias = synth.normal(2, (d,), std=0.1).astype(np.float16)
    xd, wd, bd = dev(x), dev(w), dev(bias)
    yd = ops.tensor_causal_conv1d(xd, wd, bd)
    got = host(yd).astype(np.float32)
    want = oracle.tensor_causal_conv1d(oracle.cvt_f16_to_f32(x), oracle.cvt_f16_to_f32(w), oracle.cvt_f16_to_f32(bias),
                                       threads=16)
    assert scaled_rel_err(got, want, 1.0) <= TOL_F16_ROWOPS
    assert rel_l2(got, want) <= 1e-3
    # causality at full size: perturbing one sample changes that row from there on, 4 samples long
    xd2 = xd.clone()
    xd2[2, 1234, 2047] += 1.0
    yd2 = ops.tensor_causal_conv1d(xd2, wd, bd)
    diff = (yd2 != yd).nonzero().cpu().numpy()
    assert len(diff) > 0 and np.all(diff[:, 0] == 2) and np.all(diff[:, 1] == 1234)
    assert diff[:, 2].min() >= 2047 and diff[:, 2].max() <= 2050


def test_conv1d_empty_and_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    x = torch.zeros((2, 3, 8), device="cuda", dtype=torch.float32)
    w = torch.zeros((3, 4), device="cuda", dtype=torch.float32)
    b = torch.zeros((3,), device="cuda", dtype=torch.float32)
    y = torch.full((2, 3, 8), 3.0, device="cuda", dtype=torch.float32)
    f = lib.anygpu_causal_conv1d_silu_f32
    assert f(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 2, 3, 8, 5, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 2, 3, 8, 0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(x.data_ptr(), None, b.data_ptr(), y.data_ptr(), 2, 3, 8, 4, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 2, -3, 8, 4, None) == capi.ANYGPU_ERR_BAD_SHAPE
    assert f(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 0, 3, 8, 4, None) == capi.ANYGPU_OK
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())
    with pytest.raises(ValueError):
        ops.tensor_causal_conv1d(x, torch.zeros((3, 5), device="cuda"), b)   # the reference's width assert


# =============================================================================================
# Mamba2 neighbours of the convolution: decode step, gated RMS norm
# =============================================================================================

@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("b,d,width", [(1, 1, 1), (2, 5, 4), (3, 300, 3), (4, 4224, 4), (1, 257, 2)])
def test_conv1d_update_steps_match_whole_sequence(ops, oracle, dtype, b, d, width):
    import torch
    np_dt = np.float16 if dtype == "f16" else np.float32
    s = 9
    x = synth.normal(b + d, (b, d, s)).astype(np_dt)
    w = (synth.normal(1, (d, width)) * np.float32(0.5)).astype(np_dt)
    bias = (synth.normal(2, (d,)) * np.float32(0.1)).astype(np_dt)
    up = (lambda a: oracle.cvt_f16_to_f32(a)) if dtype == "f16" else (lambda a: a)
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    state = torch.zeros((b, d, width - 1), dtype=torch.float16 if dtype == "f16" else torch.float32, device="cuda")
    ref_state = np.zeros((b, d, width - 1), dtype=np.float32)
    dw, db = dev(w), dev(bias)
    for t in range(s):
        got = host(ops.tensor_causal_conv1d_update(dev(x[:, :, t]), state, dw, db)).astype(np.float32)
        want, ref_state = oracle.causal_conv1d_update(up(x[:, :, t]), ref_state, up(w), up(bias))
        assert scaled_rel_err(got, want, 1.0) <= tol, t
        assert np.array_equal(host(state).astype(np.float32), ref_state)         # the state is a copy of samples: exact
    # and the steps together are the whole-sequence kernel
    whole = host(ops.tensor_causal_conv1d(dev(x), dw, db)).astype(np.float32)
    want_last = oracle.tensor_causal_conv1d(up(x), up(w), up(bias))[:, :, -1]
    assert scaled_rel_err(whole[:, :, -1], want_last, 1.0) <= tol
    assert scaled_rel_err(got, whole[:, :, -1], 1.0) <= tol


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 7), (5, 64), (4, 1000), (6, 1024), (3, 2048), (2, 4096), (2, 8192),
                                       (2, 8200), (1, 16384), (2, 20000), (9, 4104),
                                       # short rows sharing a block (16 lanes or a wave per row), rows walked twice
                                       (1000, 64), (300, 128), (77, 256), (501, 32), (130, 512), (45, 1000), (19, 96),
                                       (3, 50000), (2, 131072), (2, 16392)])
def test_gated_rmsnorm_shapes(ops, oracle, dtype, rows, cols):
    np_dt = np.float16 if dtype == "f16" else np.float32
    eps = 1e-5
    x = synth.normal(rows + cols, (rows, cols)).astype(np_dt)
    z = (synth.normal(cols, (rows, cols)) * np.float32(2.0)).astype(np_dt)
    w = synth.uniform(3, (cols,), 0.5, 1.5).astype(np_dt)
    up = (lambda a: oracle.cvt_f16_to_f32(a)) if dtype == "f16" else (lambda a: a)
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    got = host(ops.tensor_zamba_gated_rmsnorm(dev(x), dev(z), dev(w), cols, eps)).astype(np.float32)
    want = oracle.zamba_gated_rmsnorm(up(x), up(z), up(w), eps)
    assert scaled_rel_err(got, want, 1.0) <= tol                      # outputs have unit mean square times w ~ 1
    plain = host(ops.tensor_rms_norm(dev(x), dev(w), eps, zero_centered=True)).astype(np.float32)
    assert scaled_rel_err(plain, oracle.tensor_rms_norm(up(x), up(w), eps, zero_centered=True), 1.0) <= tol


def test_gated_rmsnorm_reference_case_group_4096(ops, oracle):
    # tests/zamba2_tests.cpp:458-476: eps 1e-5, group size 4096 = the row; rows of a [1, 70, 4096] activation
    x, z = synth.normal(1, (1, 70, 4096)), synth.normal(2, (1, 70, 4096))
    w = synth.uniform(3, (4096,), 0.5, 1.5)
    got = host(ops.tensor_zamba_gated_rmsnorm(dev(x), dev(z), dev(w), 4096, 1e-5))
    want = oracle.zamba_gated_rmsnorm(x, z, w, 1e-5)
    ok, worst = oracle.compare_data_buffers(got, want)                # the reference's own gate: abs 1e-3
    assert ok, worst
    assert scaled_rel_err(got, want, 1.0) <= TOL_F32
    # closed gate: silu(0) = 0, every output is exactly 0
    assert not host(ops.tensor_zamba_gated_rmsnorm(dev(x), dev(np.zeros_like(z)), dev(w), 4096, 1e-5)).any()


def test_mamba2_neighbours_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    x = torch.zeros((2, 8), device="cuda")
    y = torch.full((2, 8), 3.0, device="cuda")
    w = torch.ones((8,), device="cuda")
    f = lib.anygpu_gated_rmsnorm_f32
    assert f(x.data_ptr(), None, None, y.data_ptr(), 2, 8, 1e-5, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(x.data_ptr(), None, w.data_ptr(), y.data_ptr(), 2, -8, 1e-5, 0, None) == capi.ANYGPU_ERR_BAD_SHAPE
    assert f(x.data_ptr(), None, w.data_ptr(), y.data_ptr(), 2, 8, -1.0, 0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(x.data_ptr(), None, w.data_ptr(), y.data_ptr(), 0, 8, 1e-5, 0, None) == capi.ANYGPU_OK
    g = lib.anygpu_causal_conv1d_silu_update_f32
    wt = torch.ones((8, 4), device="cuda")
    assert g(x.data_ptr(), None, wt.data_ptr(), w.data_ptr(), y.data_ptr(), 2, 8, 4, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert g(x.data_ptr(), x.data_ptr(), wt.data_ptr(), w.data_ptr(), y.data_ptr(), 2, 8, 5, None) == capi.ANYGPU_ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())
    with pytest.raises(ValueError):
        ops.tensor_causal_conv1d_update(x, torch.zeros((2, 8, 2), device="cuda"), wt, w)


# =============================================================================================
# GEMM
# =============================================================================================

def test_mm_f32_reference_cases_integer_inputs_exact(ops, oracle):
    # tests/tests.cpp:94-135: crt_random_tensor inputs (integers 0..10): sums are exact in float32
    for (m, k, n) in [(40, 30, 50), (640, 1280, 320)]:
        a = synth.integers(11, (m, k), 0, 10)
        b = synth.integers(18, (k, n), 0, 10)
        got = host(ops.tensor_mm(dev(a), dev(b)))
        want = mm_want(oracle, a, b)
        assert np.array_equal(got, want)
        assert np.array_equal(got.astype(np.int64), exact_int_product(a, b))


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (3, 5, 7), (128, 16, 128), (128, 48, 256), (130, 17, 129),
                                   (256, 256, 256), (77, 300, 515), (512, 100, 64),
                                   # 16-byte aligned rows, ragged extents: vector accesses with clamped rows and guarded ends
                                   (100, 36, 72), (130, 20, 260), (257, 100, 516), (1000, 304, 520), (60, 4, 4)])
def test_mm_f32_shapes_and_layouts(ops, oracle, layout, m, k, n):
    from anygpu_amd import capi
    a = synth.uniform(m + k, (m, k))
    if layout == "row":
        b = synth.uniform(k + n, (k, n))
        got = host(ops.tensor_mm(dev(a), dev(b)))
        want = mm_want(oracle, a, b)
    else:
        bt = synth.uniform(k + n, (n, k))
        got = host(ops.tensor_mm(dev(a), dev(bt), b_layout=capi.B_COL_MAJOR))
        want = mm_want(oracle, a, bt.T)
    floor = math.sqrt(k) / 3.0          # sigma_a * sigma_b * sqrt(K) for U(-1, 1): sigma^2 = 1/3
    assert scaled_rel_err(got, want, floor) <= TOL_F32


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(128, 2304, 2048), (65, 1000, 130), (100, 4096, 72), (200, 1024, 516), (70, 515, 33),
                                   (512, 9216, 256)])
def test_mm_f32_few_tiles_split_along_k(ops, oracle, layout, m, k, n):
    # products whose tiles would not fill the chip are cut along K and merged; the cut is invisible in the result
    from anygpu_amd import capi
    a = synth.uniform(m + k, (m, k))
    b = synth.uniform(k + n, (k, n))
    want = mm_want(oracle, a, b)
    da = dev(a)
    db = dev(b) if layout == "row" else dev(np.ascontiguousarray(b.T))
    lay = capi.B_ROW_MAJOR if layout == "row" else capi.B_COL_MAJOR
    got = host(ops.tensor_mm(da, db, b_layout=lay))
    assert scaled_rel_err(got, want, math.sqrt(k) / 3.0) <= TOL_F32
    assert np.array_equal(got, host(ops.tensor_mm(da, db, b_layout=lay)))
    bias = synth.uniform(9, (n,))
    got = host(ops.tensor_gemm(da, db, dev(bias), b_layout=lay))
    assert scaled_rel_err(got, want + bias, math.sqrt(k) / 3.0) <= TOL_F32
    ai, bi = synth.integers(1, (m, k), -4, 4), synth.integers(2, (k, n), -4, 4)
    dbi = dev(bi) if layout == "row" else dev(np.ascontiguousarray(bi.T))
    assert np.array_equal(host(ops.tensor_mm(dev(ai), dbi, b_layout=lay)), mm_want(oracle, ai, bi))
    if layout == "row":
        got = host(ops.tensor_mm(dev(np.ascontiguousarray(a.T)), db, a_layout=capi.A_COL_MAJOR))
        assert scaled_rel_err(got, want, math.sqrt(k) / 3.0) <= TOL_F32


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(520, 512, 9300), (1024, 640, 4608 + 128), (300, 1024, 11000)])
def test_mm_f32_whole_rounds_and_a_rest(ops, oracle, layout, m, k, n):
    # more big tiles than one round of blocks but not a whole number of rounds: the columns of the whole rounds and
    # the rest (cut along K where that pays) are separate launches; bias and softcap reach both parts
    from anygpu_amd import capi
    a = synth.uniform(m + k, (m, k))
    b = synth.uniform(k + n, (k, n))
    bias = synth.uniform(5, (n,))
    want = mm_want(oracle, a, b)
    da = dev(a)
    db = dev(b) if layout == "row" else dev(np.ascontiguousarray(b.T))
    lay = capi.B_ROW_MAJOR if layout == "row" else capi.B_COL_MAJOR
    got = host(ops.tensor_mm(da, db, b_layout=lay))
    assert scaled_rel_err(got, want, math.sqrt(k) / 3.0) <= TOL_F32
    got = host(ops.tensor_gemm(da, db, dev(bias), b_layout=lay))
    assert scaled_rel_err(got, want + bias, math.sqrt(k) / 3.0) <= TOL_F32
    if layout == "col":
        got = host(ops.tensor_gemma_linear_softcap(da.reshape(1, m, k), db, 30.0))[0]
        ref = softcap_head_want(oracle, a.reshape(1, m, k), np.ascontiguousarray(b.T), 30.0)[0]
        assert scaled_rel_err(got, ref, math.sqrt(k) / 3.0) <= TOL_F32


def test_mm_f32_transposed_left_operand(ops, oracle):
    # the layout of the reference's last fp32 rung: A handed over as [K, M]
    from anygpu_amd import capi
    for (m, k, n) in [(128, 64, 128), (100, 37, 61), (256, 272, 384), (100, 36, 72), (260, 300, 132)]:
        a = synth.uniform(m * 7 + k, (m, k))
        b = synth.uniform(k * 5 + n, (k, n))
        at = np.ascontiguousarray(a.T)
        got = host(ops.tensor_mm(dev(at), dev(b), a_layout=capi.A_COL_MAJOR))
        want = mm_want(oracle, a, b)
        assert scaled_rel_err(got, want, math.sqrt(k) / 3.0) <= TOL_F32
        bt = np.ascontiguousarray(b.T)
        got2 = host(ops.tensor_mm(dev(at), dev(bt), a_layout=capi.A_COL_MAJOR, b_layout=capi.B_COL_MAJOR))
        assert scaled_rel_err(got2, want, math.sqrt(k) / 3.0) <= TOL_F32


def test_gemm_f32_bias_and_padded_leading_dimensions(ops, oracle):
    import torch
    from anygpu_amd import capi
    x = synth.integers(1, (50, 70), 0, 10)
    w = synth.integers(2, (70, 90), 0, 10)
    b = synth.integers(3, (90,), 0, 10)
    got = host(ops.tensor_gemm(dev(x), dev(w), dev(b)))
    assert np.array_equal(got, oracle.tensor_gemm(x, w, b))
    # operands living inside wider buffers
    abuf, bbuf = synth.uniform(4, (64, 200)), synth.uniform(5, (96, 300))
    cbuf = torch.full((64, 400), -1.0, device="cuda")
    ops.tensor_mm(dev(abuf)[:, :96], dev(bbuf)[:, :256], out=cbuf[:, :256])
    got = host(cbuf)
    want = oracle.tensor_mm(np.ascontiguousarray(abuf[:, :96]), np.ascontiguousarray(bbuf[:, :256]))
    assert scaled_rel_err(got[:, :256], want, math.sqrt(96) / 3.0) <= TOL_F32
    assert np.all(got[:, 256:] == -1.0)


def test_mm_f32_config_2048_cubed(ops, oracle):
    n = 2048
    a = synth.uniform(0, (n, n))
    b = synth.uniform(1, (n, n))
    got = host(ops.tensor_mm(dev(a), dev(b)))
    idx = sample_rows(n, 24, seed=2)
    want = np.stack([oracle.tensor_mm(a[r:r + 1], b)[0] for r in idx])
    assert scaled_rel_err(got[idx], want, math.sqrt(n) / 3.0) <= TOL_F32
    # every row and column through a checksum: C @ 1 = A @ (B @ 1), 1^T C = (1^T A) B  (float64 on the host)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64).sum(axis=1) - a64 @ b64.sum(axis=1))) < 1e-4 * n
    assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - a64.sum(axis=0) @ b64)) < 1e-4 * n


def test_mm_f16_small_integer_inputs_bit_exact(ops, oracle):
    # integers in {-2..2} and K <= 256: every partial sum is an integer of magnitude <= 1024, exact in
    # fp32 and exactly representable in the fp16 output, whatever the tiling or summation order
    from anygpu_amd import capi
    for (m, k, n) in [(64, 64, 64), (256, 256, 256), (512, 128, 768), (100, 200, 60), (33, 17, 65)]:
        a = synth.integers(m, (m, k), -2, 2, dtype=np.float16)
        bt = synth.integers(n, (n, k), -2, 2, dtype=np.float16)
        want = oracle.tensor_mm(oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(bt).T)
        got_nt = host(ops.tensor_mm(dev(a), dev(bt), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
        assert np.array_equal(got_nt, want), (m, k, n, "col-major B")
        got_nn = host(ops.tensor_mm(dev(a), dev(np.ascontiguousarray(bt.T)))).astype(np.float32)
        assert np.array_equal(got_nn, want), (m, k, n, "row-major B")


def test_mm_f16_reference_case_640x1280_1280x320(ops, oracle):
    # tests/tests.cpp:138-164: N(0,1) fp16 operands, CPU fp32 matmul of the up-cast inputs, rel-L2 <= 0.01
    a = synth.normal(11, (640, 1280)).astype(np.float16)
    b = synth.normal(18, (1280, 320)).astype(np.float16)
    got = host(ops.tensor_mm(dev(a), dev(b))).astype(np.float32)
    want = mm_want(oracle, oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(b))
    ok, val = oracle.compare_data_buffers_l2(got, want, 0.01)
    assert ok, val
    assert scaled_rel_err(got, want, math.sqrt(1280)) <= TOL_F16_GEMM


@pytest.mark.parametrize("m,k,n", [(256, 64, 256), (256, 128, 512), (768, 192, 1024), (1024, 1024, 1024),
                                   (128, 64, 128), (384, 320, 640), (128, 128, 1152), (2304, 192, 256),
                                   (64, 64, 64), (640, 1280, 320), (192, 448, 64), (320, 64, 1088)])
def test_mm_f16_tile_kernel_shapes(ops, oracle, m, k, n):
    from anygpu_amd import capi
    a = synth.uniform(m + 1, (m, k)).astype(np.float16)
    bt = synth.uniform(n + 2, (n, k)).astype(np.float16)
    want = mm_want(oracle, oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(bt).T)
    got = host(ops.tensor_mm(dev(a), dev(bt), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    assert scaled_rel_err(got, want, math.sqrt(k) / 3.0) <= TOL_F16_GEMM
    assert rel_l2(got, want) <= 1e-2
    # the same product with B in the reference layout [K, N] (transposing LDS reads)
    got_kn = host(ops.tensor_mm(dev(a), dev(np.ascontiguousarray(bt.T)))).astype(np.float32)
    assert scaled_rel_err(got_kn, want, math.sqrt(k) / 3.0) <= TOL_F16_GEMM
    # both layouts feed the same MFMA sequence: identical results
    assert np.array_equal(got_kn, got)


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(100, 64, 72), (130, 128, 264), (257, 192, 1000), (1000, 256, 520), (300, 64, 8),
                                   (65, 64, 136), (9, 128, 4096), (2047, 64, 2056), (520, 320, 248),
                                   (128, 72, 128), (256, 200, 256), (100, 136, 72), (1024, 1000, 1024), (300, 88, 520)])
def test_mm_f16_ragged_shapes_through_tile_kernels(ops, oracle, layout, m, k, n):
    # K >= 64 and K, N multiples of 8: the MFMA tile kernels with clamped operand rows, guarded stores and,
    # when K is not a multiple of 64, a tail multiplied from registers
    import torch
    from anygpu_amd import capi
    a = synth.uniform(m + k, (m, k)).astype(np.float16)
    b = synth.uniform(k + n, (k, n)).astype(np.float16)
    want = mm_want(oracle, oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(b))
    # the result sits inside a larger buffer: nothing outside [m, n] may be touched
    cbuf = torch.full((m + 3, n + 16), -7.0, device="cuda", dtype=torch.float16)
    if layout == "row":
        ops.tensor_mm(dev(a), dev(b), out=cbuf[:m, :n])
    else:
        ops.tensor_mm(dev(a), dev(np.ascontiguousarray(b.T)), out=cbuf[:m, :n], b_layout=capi.B_COL_MAJOR)
    got = host(cbuf).astype(np.float32)
    assert scaled_rel_err(got[:m, :n], want, math.sqrt(k) / 3.0) <= TOL_F16_GEMM
    assert np.all(got[m:, :] == -7.0) and np.all(got[:, n:] == -7.0)


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(128, 9216, 2304), (100, 1032, 72), (256, 4104, 520), (65, 2304, 2048), (300, 1024, 64),
                                   (512, 8200, 256)])
def test_mm_f16_few_tiles_split_along_k(ops, oracle, layout, m, k, n):
    # fewer blocks than CUs and a deep K: ranges of K write fp32 planes that a merge kernel adds and rounds once
    from anygpu_amd import capi
    a = synth.uniform(m + k, (m, k)).astype(np.float16)
    b = synth.uniform(k + n, (k, n)).astype(np.float16)
    want = mm_want(oracle, oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(b))
    da = dev(a)
    db = dev(b) if layout == "row" else dev(np.ascontiguousarray(b.T))
    lay = capi.B_ROW_MAJOR if layout == "row" else capi.B_COL_MAJOR
    got = host(ops.tensor_mm(da, db, b_layout=lay))
    assert scaled_rel_err(got.astype(np.float32), want, math.sqrt(k) / 3.0) <= TOL_F16_GEMM
    assert np.array_equal(got, host(ops.tensor_mm(da, db, b_layout=lay)))
    ai, bi = synth.integers(1, (m, k), -2, 2).astype(np.float16), synth.integers(2, (k, n), -2, 2).astype(np.float16)
    dbi = dev(bi) if layout == "row" else dev(np.ascontiguousarray(bi.T))
    want_i = mm_want(oracle, ai.astype(np.float32), bi.astype(np.float32))
    assert np.array_equal(host(ops.tensor_mm(dev(ai), dbi, b_layout=lay)).astype(np.float32), want_i.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(4096, 128, 5120), (2100, 64, 8000), (4352, 64, 4352)])
def test_mm_f16_whole_rounds_and_a_rest(ops, oracle, layout, m, k, n):
    # more 256 x 256 tiles than one round of blocks but not a whole number of rounds: two launches, divided by columns
    from anygpu_amd import capi
    a = synth.integers(m + k, (m, k), -2, 2).astype(np.float16)
    b = synth.integers(k + n, (k, n), -2, 2).astype(np.float16)
    want = mm_want(oracle, a.astype(np.float32), b.astype(np.float32))
    db = dev(b) if layout == "row" else dev(np.ascontiguousarray(b.T))
    lay = capi.B_ROW_MAJOR if layout == "row" else capi.B_COL_MAJOR
    got = host(ops.tensor_mm(dev(a), db, b_layout=lay)).astype(np.float32)
    assert np.array_equal(got, want)


def test_mm_f16_ragged_integer_inputs_bit_exact_and_batched(ops, oracle):
    from anygpu_amd import capi
    a = synth.integers(1, (200, 128), -4, 4).astype(np.float16)
    b = synth.integers(2, (128, 328), -4, 4).astype(np.float16)
    want = oracle.tensor_mm(a.astype(np.float32), b.astype(np.float32))
    assert np.array_equal(host(ops.tensor_mm(dev(a), dev(b))).astype(np.float32), want)
    assert np.array_equal(host(ops.tensor_mm(dev(a), dev(np.ascontiguousarray(b.T)), b_layout=capi.B_COL_MAJOR)).astype(np.float32), want)
    # a batch of ragged products (attention shapes: 100 queries x 72 keys, d = 64)
    q = synth.normal(3, (6, 100, 64)).astype(np.float16)
    kk = synth.normal(4, (6, 72, 64)).astype(np.float16)
    got = host(ops.tensor_mm_batched(dev(q), dev(kk), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    for i in range(6):
        w = oracle.tensor_mm(oracle.cvt_f16_to_f32(q[i]), oracle.cvt_f16_to_f32(kk[i]).T)
        assert scaled_rel_err(got[i], w, math.sqrt(64)) <= TOL_F16_GEMM


def test_mm_f16_config_4096_cubed_col_major_b(ops, oracle):
    from anygpu_amd import capi
    n = 4096
    a = synth.uniform(0, (n, n)).astype(np.float16)
    bt = synth.uniform(1, (n, n)).astype(np.float16)      # B stored [N, K]
    got = host(ops.tensor_mm(dev(a), dev(bt), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    a32, bt32 = oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(bt)
    idx = sample_rows(n, 24, seed=3)
    want = np.stack([oracle.tensor_mm(a32[r:r + 1], bt32.T)[0] for r in idx])
    floor = math.sqrt(n) / 3.0
    assert scaled_rel_err(got[idx], want, floor) <= TOL_F16_GEMM
    assert rel_l2(got[idx], want) <= 1e-2
    # checksums over every row and every column (fp16 output rounding: 2^-11 relative per element)
    a64, b64 = a32.astype(np.float64), bt32.astype(np.float64)
    row_sum = a64 @ b64.sum(axis=0)
    col_sum = a64.sum(axis=0) @ b64.T
    g64 = got.astype(np.float64)
    tol = n * floor * 2.0 ** -11 * 4
    assert np.max(np.abs(g64.sum(axis=1) - row_sum)) < tol
    assert np.max(np.abs(g64.sum(axis=0) - col_sum)) < tol


@pytest.mark.parametrize("m,n,k,pad", [(4096, 4096, 64, 0), (4096, 4096, 128, 0), (4096, 4096, 192, 8), (2048, 8192, 320, 0),
                                       (8192, 2048, 256, 72), (3840, 4352, 64, 0), (4000, 3896, 128, 0), (3841, 4104, 64, 8),
                                       (4095, 4088, 192, 0), (3969, 3848, 64, 0)])
def test_mm_f16_whole_256_tiles_integer_inputs_exact(ops, m, n, k, pad):
    # Shapes of 256 x 256 tiles with k-contiguous weights take the four-wave kernel whose main loop is an assembly
    # block: one slab (K = 64), two, an odd number, padded leading dimensions, a tile count that is no multiple of the
    # 8 XCDs, ragged M and N (a last tile of 1 row, of 8 columns: whole waves of it read clamped rows).  Integers in -2 .. 2 with K <= 320: every sum is an integer below 2^11, exact in fp32 and in the fp16
    # result, whatever the order of summation.
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k, (m, k), -2, 2).astype(np.float16)
    bt = synth.integers(n + k + 1, (n, k), -2, 2).astype(np.float16)
    a_dev = torch.zeros((m, k + pad), dtype=torch.float16, device="cuda")
    b_dev = torch.full((n, k + pad), 7.0, dtype=torch.float16, device="cuda")      # the padding must not be read as data
    a_dev[:, :k] = dev(a)
    b_dev[:, :k] = dev(bt)
    got = host(ops.tensor_mm(a_dev[:, :k], b_dev[:, :k], b_layout=capi.B_COL_MAJOR)).astype(np.int64)
    want = exact_int_product(a, bt.T)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k,pad", [(4096, 4096, 64, 0), (4096, 4096, 128, 8), (2048, 8192, 320, 0), (3840, 4352, 192, 264),
                                       (4000, 3896, 128, 0), (3841, 4104, 64, 8), (4095, 4088, 192, 0), (3969, 3848, 64, 0)])
def test_mm_f16_256_tiles_reference_layout_integer_inputs_exact(ops, m, n, k, pad):
    # the same kernel with B stored [K, N] as the reference stores it: units of 64 k rows, transposing LDS reads, a row
    # pitch that is not the row length, a last tile of 8 columns whose other chunks are read from inside the row
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k + 2, (m, k), -2, 2).astype(np.float16)
    b = synth.integers(n + k + 3, (k, n), -2, 2).astype(np.float16)
    b_dev = torch.full((k, n + pad), 7.0, dtype=torch.float16, device="cuda")
    b_dev[:, :n] = dev(b)
    got = host(ops.tensor_mm(dev(a), b_dev[:, :n], b_layout=capi.B_ROW_MAJOR)).astype(np.int64)
    want = exact_int_product(a, b)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k,pad,span", [(2048, 2048, 192, 0, 2), (1000, 2000, 128, 8, 2), (2048, 4096, 64, 0, 2), (1100, 4000, 320, 0, 2),
                                            (520, 6152, 256, 0, 2), (128, 128, 64, 0, 2), (512, 2304, 9216, 0, 1), (300, 1000, 4096, 72, 1),
                                            (2048, 1024, 2048, 0, 1)])
def test_mm_f16_smaller_four_wave_tiles_integer_inputs_exact(ops, m, n, k, pad, span):
    # products that do not fill the chip with 256 x 256 tiles: the four-wave kernels with 256 x 128 and 128 x 128 tiles,
    # whole and ragged, one slab and several, and cut along K into fp32 planes (the deep ones).  Integer operands whose
    # sums stay below 2^11 in magnitude are exact in fp32 and in the fp16 result in any order of summation.
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k + 4, (m, k), -span, span).astype(np.float16)
    bt = synth.integers(n + k + 5, (n, k), -span, span).astype(np.float16)
    a_dev = torch.full((m, k + pad), 7.0, dtype=torch.float16, device="cuda")
    b_dev = torch.full((n, k + pad), 7.0, dtype=torch.float16, device="cuda")
    a_dev[:, :k] = dev(a)
    b_dev[:, :k] = dev(bt)
    got = host(ops.tensor_mm(a_dev[:, :k], b_dev[:, :k], b_layout=capi.B_COL_MAJOR)).astype(np.int64)
    want = exact_int_product(a, bt.T)
    assert np.abs(want).max() < 2048
    assert np.array_equal(got, want)


@pytest.mark.parametrize("layout,m,n,k,a_off,b_off,pad", [
    ("row", 1024, 1028, 512, 0, 0, 0),       # [K, N] weights with N no multiple of 8
    ("row", 512, 1000, 1027, 0, 0, 0),       # K no multiple of 8: both operands
    ("col", 600, 1000, 1027, 0, 0, 0),
    ("col", 512, 1024, 512, 1, 0, 0),        # A starts at an odd element
    ("col", 512, 1024, 512, 0, 3, 0),        # B starts at an odd element
    ("col", 512, 1024, 512, 0, 0, 3),        # row pitches no multiple of 8
    ("row", 700, 1096, 520, 5, 1, 1),        # everything at once
    ("col", 2048, 2052, 1000, 1, 1, 0),
])
def test_mm_f16_operands_the_tile_kernels_cannot_fetch_are_copied(ops, layout, m, n, k, a_off, b_off, pad):
    # operands at odd addresses, with odd row pitches, a K or (weights stored [K, N]) an N that is no multiple of 8, in
    # products big enough to pay for it: aligned zero-padded copies in the stream's workspace, then the ordinary
    # kernels.  Integer operands: exact whatever the summation order.  Guard values around every buffer: the copies must
    # not read them as data, the product must not write outside the result.
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k + 6, (m, k), -1, 1).astype(np.float16)
    b = synth.integers(n + k + 7, (k, n), -1, 1).astype(np.float16)
    a_flat = torch.full((a_off + m * (k + pad) + 8,), 9.0, dtype=torch.float16, device="cuda")
    a_view = a_flat[a_off:a_off + m * (k + pad)].view(m, k + pad)[:, :k]
    a_view.copy_(dev(a))
    rows, cols = (k, n) if layout == "row" else (n, k)
    b_flat = torch.full((b_off + rows * (cols + pad) + 8,), 9.0, dtype=torch.float16, device="cuda")
    b_view = b_flat[b_off:b_off + rows * (cols + pad)].view(rows, cols + pad)[:, :cols]
    b_view.copy_(dev(b if layout == "row" else np.ascontiguousarray(b.T)))
    cbuf = torch.full((m + 2, n + 9), -7.0, device="cuda", dtype=torch.float16)
    ops.tensor_mm(a_view, b_view, out=cbuf[:m, :n], b_layout=capi.B_ROW_MAJOR if layout == "row" else capi.B_COL_MAJOR)
    got = host(cbuf).astype(np.int64)
    want = exact_int_product(a, b)
    assert np.abs(want).max() < 2048
    assert np.array_equal(got[:m, :n], want)
    assert np.all(got[m:, :] == -7) and np.all(got[:, n:] == -7)


@pytest.mark.parametrize("layout,m,n,k,a_off,b_off,pad", [
    ("row", 2047, 2047, 2047, 0, 0, 0), ("col", 1023, 1025, 1030, 0, 0, 0), ("row", 1024, 1024, 512, 1, 0, 0),
    ("col", 1024, 1024, 512, 0, 3, 0), ("row", 700, 1096, 720, 2, 1, 1), ("col", 1024, 1024, 512, 0, 0, 3),
    ("row", 1000, 1000, 1000, 0, 0, 0), ("col", 2044, 2044, 520, 0, 0, 0),
])
def test_mm_f32_operands_at_odd_addresses_are_copied(ops, layout, m, n, k, a_off, b_off, pad):
    # fp32 operands with odd starts or row pitches, in products big enough to pay for it: aligned copies in the stream's
    # workspace, then the ordinary kernels (C keeps its own alignment).  Integer operands: every sum exact in fp32.
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k + 8, (m, k), -3, 3).astype(np.float32)
    b = synth.integers(n + k + 9, (k, n), -3, 3).astype(np.float32)
    a_flat = torch.full((a_off + m * (k + pad) + 8,), 9.0, dtype=torch.float32, device="cuda")
    a_view = a_flat[a_off:a_off + m * (k + pad)].view(m, k + pad)[:, :k]
    a_view.copy_(dev(a))
    rows, cols = (k, n) if layout == "row" else (n, k)
    b_flat = torch.full((b_off + rows * (cols + pad) + 8,), 9.0, dtype=torch.float32, device="cuda")
    b_view = b_flat[b_off:b_off + rows * (cols + pad)].view(rows, cols + pad)[:, :cols]
    b_view.copy_(dev(b if layout == "row" else np.ascontiguousarray(b.T)))
    cbuf = torch.full((m + 2, n + 5), -7.0, device="cuda", dtype=torch.float32)
    ops.tensor_mm(a_view, b_view, out=cbuf[:m, :n], b_layout=capi.B_ROW_MAJOR if layout == "row" else capi.B_COL_MAJOR)
    got = host(cbuf).astype(np.int64)
    want = exact_int_product(a, b)
    assert np.array_equal(got[:m, :n], want)
    assert np.all(got[m:, :] == -7) and np.all(got[:, n:] == -7)


@pytest.mark.parametrize("m,n,k,pad,span", [(2048, 2048, 192, 0, 2), (1000, 2000, 128, 8, 2), (2048, 4096, 64, 0, 2), (1100, 4000, 320, 0, 2),
                                            (520, 6152, 256, 16, 2), (128, 128, 64, 0, 2), (512, 2304, 9216, 0, 1), (300, 1000, 4096, 72, 1),
                                            (2048, 1024, 2048, 0, 1)])
def test_mm_f16_smaller_four_wave_tiles_reference_layout_exact(ops, m, n, k, pad, span):
    # the same products with B stored [K, N]: units of 64 k rows x 128 n, transposing reads, a row pitch that is not the
    # row length, last tiles of 8 columns, cuts along K that step down the rows of B
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k + 10, (m, k), -span, span).astype(np.float16)
    b = synth.integers(n + k + 11, (k, n), -span, span).astype(np.float16)
    b_dev = torch.full((k, n + pad), 7.0, dtype=torch.float16, device="cuda")
    b_dev[:, :n] = dev(b)
    got = host(ops.tensor_mm(dev(a), b_dev[:, :n], b_layout=capi.B_ROW_MAJOR)).astype(np.int64)
    want = exact_int_product(a, b)
    assert np.abs(want).max() < 2048
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k,pad", [(128, 128, 32, 0), (2048, 2048, 64, 0), (2048, 2048, 96, 4), (1000, 2000, 160, 8), (130, 4100, 32, 0),
                                       (2048, 1024, 2048, 0), (256, 2304, 9216, 0), (3000, 1031, 64, 1)])
def test_mm_f32_four_wave_kernel_integer_inputs_exact(ops, m, n, k, pad):
    # fp32 products of k-contiguous operands in whole 32-deep slabs take the four-wave kernel whose main loop is an
    # assembly block: one slab, two, three, padded pitches, ragged M and N, a C with an odd pitch, deep K cut into planes.
    # Integer operands: every sum is exact in fp32 whatever the order.
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + k + 12, (m, k), -3, 3).astype(np.float32)
    bt = synth.integers(n + k + 13, (n, k), -3, 3).astype(np.float32)
    a_dev = torch.full((m, k + pad), 7.0, dtype=torch.float32, device="cuda")
    b_dev = torch.full((n, k + pad), 7.0, dtype=torch.float32, device="cuda")
    a_dev[:, :k] = dev(a)
    b_dev[:, :k] = dev(bt)
    cbuf = torch.full((m + 1, n + 3), -7.0, device="cuda", dtype=torch.float32)
    ops.tensor_mm(a_dev[:, :k], b_dev[:, :k], out=cbuf[:m, :n], b_layout=capi.B_COL_MAJOR)
    got = host(cbuf).astype(np.int64)
    want = exact_int_product(a, bt.T)
    assert np.array_equal(got[:m, :n], want)
    assert np.all(got[m:, :] == -7) and np.all(got[:, n:] == -7)


@pytest.mark.parametrize("m,n,k,pad", [(128, 128, 32, 0), (2048, 2048, 64, 0), (2048, 2048, 96, 4), (1000, 2000, 160, 8), (130, 4100, 32, 0),
                                       (2048, 1024, 2048, 0), (256, 2304, 9216, 0), (3000, 1032, 64, 4), (64, 64, 32, 0), (500, 260, 128, 0)])
def test_mm_f32_four_wave_kernel_reference_layout_exact(ops, m, n, k, pad):
    # the same kernels with B stored [K, N] as the reference stores it: units of 32 k rows, a lane fetches its k down a
    # column, the chunks of the upper sixteen rows stored with a flipped index bit; pitches that are not the row length,
    # last tiles of 4 columns, deep K cut into planes that step down the rows of B
    import torch
    a = synth.integers(m + k + 14, (m, k), -3, 3).astype(np.float32)
    b = synth.integers(n + k + 15, (k, n), -3, 3).astype(np.float32)
    b_dev = torch.full((k, n + pad), 7.0, dtype=torch.float32, device="cuda")
    b_dev[:, :n] = dev(b)
    cbuf = torch.full((m + 1, n + 3), -7.0, device="cuda", dtype=torch.float32)
    ops.tensor_mm(dev(a), b_dev[:, :n], out=cbuf[:m, :n])
    got = host(cbuf).astype(np.int64)
    want = exact_int_product(a, b)
    assert np.array_equal(got[:m, :n], want)
    assert np.all(got[m:, :] == -7) and np.all(got[:, n:] == -7)


def test_mm_f16_whole_256_tiles_batched(ops, oracle):
    # four products of 2048 x 2048 x 128 in one launch: 256 tiles of 256 x 256, the four-wave kernel over blockIdx.y
    from anygpu_amd import capi
    batch, n, k = 4, 2048, 128
    a = synth.uniform(5, (batch, n, k)).astype(np.float16)
    bt = synth.uniform(6, (batch, n, k)).astype(np.float16)
    got = host(ops.tensor_mm_batched(dev(a), dev(bt), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    a32, bt32 = oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(bt)
    floor = math.sqrt(k) / 3.0
    for i in range(batch):
        idx = sample_rows(n, 16, seed=i)
        want = np.stack([oracle.tensor_mm(a32[i, r:r + 1], bt32[i].T)[0] for r in idx])
        assert scaled_rel_err(got[i][idx], want, floor) <= TOL_F16_GEMM
        ref64 = a32[i].astype(np.float64) @ bt32[i].astype(np.float64).T
        assert np.max(np.abs(got[i] - ref64)) <= floor * 2e-2


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", [(1, 2304, 9216), (1, 64, 8), (2, 512, 1000), (3, 2304, 2050), (4, 1000, 512),
                                   (5, 72, 70), (8, 4096, 1024), (7, 8, 3), (1, 9216, 2304), (8, 33, 64)])
def test_mm_few_rows(ops, oracle, dtype, layout, m, k, n):
    # the decode-step shapes (M <= 8) take the bandwidth-shaped kernels when alignment allows, the tile kernels otherwise
    from anygpu_amd import capi
    np_dt = np.float16 if dtype == "f16" else np.float32
    a = synth.uniform(m * 3 + k, (m, k)).astype(np_dt)
    b = synth.uniform(k * 5 + n, (k, n)).astype(np_dt)
    a32 = oracle.cvt_f16_to_f32(a) if dtype == "f16" else a
    b32 = oracle.cvt_f16_to_f32(b) if dtype == "f16" else b
    want = mm_want(oracle, a32, b32)
    if layout == "row":
        got = host(ops.tensor_mm(dev(a), dev(b)))
    else:
        got = host(ops.tensor_mm(dev(a), dev(np.ascontiguousarray(b.T)), b_layout=capi.B_COL_MAJOR))
    tol = TOL_F16_GEMM if dtype == "f16" else TOL_F32
    assert got.shape == (m, n)
    assert scaled_rel_err(got.astype(np.float32), want, math.sqrt(k) / 3.0) <= tol


def test_mm_few_rows_integer_inputs_exact_and_padded_buffers(ops, oracle):
    import torch
    from anygpu_amd import capi
    for (m, k, n) in [(1, 256, 96), (6, 128, 260)]:
        a = synth.integers(1, (m, k), -4, 4)
        b = synth.integers(2, (k, n), -4, 4)
        want = oracle.tensor_mm(a, b)
        assert np.array_equal(host(ops.tensor_mm(dev(a), dev(b))), want)
        assert np.array_equal(host(ops.tensor_mm(dev(a), dev(np.ascontiguousarray(b.T)), b_layout=capi.B_COL_MAJOR)), want)
        bias = synth.integers(3, (n,), -9, 9)
        assert np.array_equal(host(ops.tensor_gemm(dev(a), dev(b), dev(bias))), oracle.tensor_gemm(a, b, bias))
    # operands and result inside wider buffers
    abuf, bbuf = synth.uniform(4, (4, 200)), synth.uniform(5, (96, 300))
    cbuf = torch.full((4, 400), -1.0, device="cuda")
    ops.tensor_mm(dev(abuf)[:, :96], dev(bbuf)[:, :256], out=cbuf[:, :256])
    got = host(cbuf)
    want = oracle.tensor_mm(np.ascontiguousarray(abuf[:, :96]), np.ascontiguousarray(bbuf[:, :256]))
    assert scaled_rel_err(got[:, :256], want, math.sqrt(96) / 3.0) <= TOL_F32
    assert np.all(got[:, 256:] == -1.0)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("m,k,n", [(9, 2304, 9216), (16, 9216, 2304), (17, 512, 1000), (32, 2304, 2052), (12, 72, 68),
                                   (31, 264, 132), (24, 4096, 128), (10, 8, 4), (20, 1000, 130), (13, 16, 3000),
                                   (33, 2304, 2052), (64, 9216, 2304), (48, 200, 1000), (5, 2304, 4100), (57, 72, 36),
                                   (40, 520, 33000), (37, 4104, 260)])
def test_mm_row_bands(ops, oracle, dtype, m, k, n):
    # 5 <= M <= 64 against k-contiguous weights: the streaming kernels, with K split over blocks where N alone gives
    # too few tiles (the split is invisible in the result: every launch adds the partial sums in the same order)
    from anygpu_amd import capi
    np_dt = np.float16 if dtype == "f16" else np.float32
    a = synth.uniform(m * 3 + k, (m, k)).astype(np_dt)
    bt = synth.uniform(k * 5 + n, (n, k)).astype(np_dt)
    a32 = oracle.cvt_f16_to_f32(a) if dtype == "f16" else a
    b32 = np.ascontiguousarray((oracle.cvt_f16_to_f32(bt) if dtype == "f16" else bt).T)
    want = mm_want(oracle, a32, b32)
    da, db = dev(a), dev(bt)
    got = host(ops.tensor_mm(da, db, b_layout=capi.B_COL_MAJOR))
    tol = TOL_F16_GEMM if dtype == "f16" else TOL_F32
    assert got.shape == (m, n)
    assert scaled_rel_err(got.astype(np.float32), want, math.sqrt(k) / 3.0) <= tol
    again = host(ops.tensor_mm(da, db, b_layout=capi.B_COL_MAJOR))
    assert np.array_equal(got, again)


@pytest.mark.parametrize("m,k,n", [(9, 2304, 9216), (16, 9216, 2304), (17, 512, 1000), (32, 2304, 2052), (12, 72, 68),
                                   (31, 264, 132), (24, 4096, 128), (10, 8, 4), (20, 1000, 132), (13, 16, 3000),
                                   (64, 9216, 2304), (48, 200, 1000), (5, 2304, 4100), (57, 72, 36), (40, 520, 132000),
                                   (37, 4104, 260), (8, 1028, 516)])
def test_mm_f32_row_bands_n_contiguous_weights(ops, oracle, m, k, n):
    # the same bands against weights stored [K, N], the layout of the reference's linear layers
    import torch
    a = synth.uniform(m * 3 + k, (m, k))
    b = synth.uniform(k * 5 + n, (k, n))
    want = mm_want(oracle, a, b)
    da, db = dev(a), dev(b)
    got = host(ops.tensor_mm(da, db))
    assert scaled_rel_err(got, want, math.sqrt(k) / 3.0) <= TOL_F32
    assert np.array_equal(got, host(ops.tensor_mm(da, db)))
    bias = synth.uniform(7, (n,))
    got = host(ops.tensor_gemm(da, db, dev(bias)))
    assert scaled_rel_err(got, want + bias, math.sqrt(k) / 3.0) <= TOL_F32
    if m <= 40 and n <= 9216:
        ai, bi = synth.integers(1, (m, k), -4, 4), synth.integers(2, (k, n), -4, 4)
        assert np.array_equal(host(ops.tensor_mm(dev(ai), dev(bi))), mm_want(oracle, ai, bi))
        # operands and result inside wider buffers
        abuf, bbuf = torch.zeros((m, k + 8), device="cuda"), torch.zeros((k, n + 12), device="cuda")
        abuf[:, :k], bbuf[:, :n] = da, db
        cbuf = torch.full((m, n + 4), -1.0, device="cuda")
        ops.tensor_mm(abuf[:, :k], bbuf[:, :n], out=cbuf[:, :n])
        assert np.array_equal(host(cbuf[:, :n]), host(ops.tensor_mm(da, db)))
        assert bool((cbuf[:, n:] == -1.0).all())


@pytest.mark.parametrize("m,k,n", [(1, 2304, 32003), (8, 2304, 32001), (16, 512, 1001), (32, 1028, 518), (5, 64, 7), (9, 72, 5),
                                   (24, 4096, 131), (40, 520, 132002), (64, 9216, 2305), (3, 16, 4), (12, 200, 258), (33, 512, 1003),
                                   (2, 256, 1001), (4, 64, 3), (1, 1024, 50257), (3, 72, 2)])
def test_mm_row_bands_rows_of_any_length(ops, oracle, m, k, n):
    # N no multiple of four: weight rows ([K, N]) and result rows start at any element; small integers, so exact
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + 1, (m, k), -4, 4)
    b = synth.integers(n + 2, (k, n), -4, 4)
    want = mm_want(oracle, a, b)
    da, db = dev(a), dev(b)
    assert np.array_equal(host(ops.tensor_mm(da, db)), want)
    bias = synth.integers(3, (n,), -9, 9)
    assert np.array_equal(host(ops.tensor_gemm(da, db, dev(bias))), want + bias)
    # the same weights stored [N, K]: only the rows of the result are unaligned
    dbt = dev(np.ascontiguousarray(b.T))
    assert np.array_equal(host(ops.tensor_mm(da, dbt, b_layout=capi.B_COL_MAJOR)), want)
    if k % 8 == 0 and np.abs(want).max() <= 2048:      # (integers up to 2048 are exact in fp16)
        a16, bt16 = a.astype(np.float16), np.ascontiguousarray(b.T).astype(np.float16)
        assert np.array_equal(host(ops.tensor_mm(dev(a16), dev(bt16), b_layout=capi.B_COL_MAJOR)).astype(np.float32), want)
        assert np.array_equal(host(ops.tensor_mm(dev(a16), dev(b.astype(np.float16)))).astype(np.float32), want)
    # result inside a wider buffer with an odd row length: nothing beyond column n is touched
    cbuf = torch.full((m, n + 3), -1.0, device="cuda")
    ops.tensor_mm(da, db, out=cbuf[:, :n])
    assert np.array_equal(host(cbuf[:, :n]), want)
    assert bool((cbuf[:, n:] == -1.0).all())
    cbuf.fill_(-1.0)
    ops.tensor_mm(da, dbt, out=cbuf[:, :n], b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(cbuf[:, :n]), want)
    assert bool((cbuf[:, n:] == -1.0).all())


@pytest.mark.parametrize("m,k,n", [(1, 64, 131072), (8, 96, 131080), (16, 32, 200000), (17, 160, 140000), (33, 128, 131592),
                                   (48, 64, 131072), (64, 224, 132096), (8, 96, 32000), (40, 160, 65544), (64, 64, 24576),
                                   (3, 32, 100000), (20, 288, 50264), (24, 64, 65536), (32, 96, 65544)])
def test_mm_f16_row_bands_n_contiguous_weights_many_columns(ops, oracle, m, k, n):
    # few rows against [K, N] fp16 weights with the columns of an output head: the band kernel that transposes 8 x 8
    # blocks of the weights in registers, waves side by side (from about 123000 columns) or sharing their columns and
    # dividing K; small integers, so every sum is exact in fp16
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + 11, (m, k), -2, 2)
    b = synth.integers(n + 12, (k, n), -2, 2)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da, db = dev(a.astype(np.float16)), dev(b.astype(np.float16))
    got = host(ops.tensor_mm(da, db)).astype(np.float32)
    assert np.array_equal(got, want)
    # operands and result inside wider buffers: nothing beyond column n is touched
    abuf = torch.zeros((m, k + 8), device="cuda", dtype=torch.float16)
    bbuf = torch.zeros((k, n + 16), device="cuda", dtype=torch.float16)
    abuf[:, :k], bbuf[:, :n] = da, db
    cbuf = torch.full((m, n + 8), -1.0, device="cuda", dtype=torch.float16)
    ops.tensor_mm(abuf[:, :k], bbuf[:, :n], out=cbuf[:, :n])
    assert np.array_equal(host(cbuf[:, :n]).astype(np.float32), want)
    assert bool((cbuf[:, n:] == -1.0).all())
    # uniform operands against the oracle at the fp16 GEMM tolerance, and the softcap epilogue on the same sums
    au = synth.uniform(m + 13, (m, k)).astype(np.float16)
    bu = synth.uniform(n + 14, (k, n)).astype(np.float16)
    ref = mm_want(oracle, oracle.cvt_f16_to_f32(au), oracle.cvt_f16_to_f32(bu))
    dau, dbu = dev(au), dev(bu)
    got = host(ops.tensor_mm(dau, dbu)).astype(np.float32)
    assert scaled_rel_err(got, ref, math.sqrt(k) / 3.0) <= TOL_F16_GEMM
    out = torch.empty((m, n), device="cuda", dtype=torch.float16)
    lib = capi.load()
    capi.check("anygpu_gemm_f16_f32acc_softcap",
               lib.anygpu_gemm_f16_f32acc_softcap(dau.data_ptr(), dbu.data_ptr(), out.data_ptr(), m, n, k, k, n, n, capi.B_ROW_MAJOR,
                                                  2.0, torch.cuda.current_stream().cuda_stream))
    capped = oracle.softcap(ref, 2.0).reshape(m, n)
    assert scaled_rel_err(host(out).astype(np.float32), capped, 2.0 / 3.0) <= TOL_F16_GEMM


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("m,steps,n", [(3, 1, 131072), (5, 2, 125000), (8, 3, 131068), (16, 4, 196608), (13, 5, 124672),
                                       (17, 6, 131072), (32, 2, 125000), (9, 8, 262144), (40, 2, 131072), (48, 3, 125000),
                                       (64, 2, 131072),
                                       # fewer columns and a deep K: the same kernel over ranges of K, planes and a merge (fp32)
                                       (16, 128, 32000), (24, 128, 32000), (5, 96, 32004), (40, 144, 36864)])
def test_mm_row_bands_k_contiguous_weights_many_columns(ops, oracle, dtype, m, steps, n):
    # few rows against [N, K] weights with the columns of an output head: the band kernel that loads whole 128-byte
    # lines per weight row and lets lane pairs exchange halves, blocks starting at different chunks of K (an odd number
    # of 128-byte steps: all at chunk 0); the column counts give (nearly) two or more blocks of 256 columns per CU
    # of a 256-CU device, some with a ragged last block.  Row counts outside the kernel's range (fp32: 3 to 48 rows,
    # fp16: 3 to 64) check the kernels that take those.  Small integers: every sum is exact.
    import torch
    from anygpu_amd import capi
    half = dtype == "f16"
    tdt, ndt = (torch.float16, np.float16) if half else (torch.float32, np.float32)
    k = steps * (64 if half else 32)
    a = synth.integers(m + 21, (m, k), -2, 2)
    w = synth.integers(n + 22, (n, k), -2, 2)
    want = mm_want(oracle, a, w.T)
    assert np.abs(want).max() <= 2048
    da, dw = dev(a.astype(ndt)), dev(w.astype(ndt))
    got = host(ops.tensor_mm(da, dw, b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    assert np.array_equal(got, want)
    # operands and result inside wider buffers: nothing beyond column n is touched
    pad = 8 if half else 4
    abuf = torch.zeros((m, k + pad), device="cuda", dtype=tdt)
    wbuf = torch.zeros((n, k + 2 * pad), device="cuda", dtype=tdt)
    abuf[:, :k], wbuf[:, :k] = da, dw
    cbuf = torch.full((m, n + 4), -1.0, device="cuda", dtype=tdt)
    ops.tensor_mm(abuf[:, :k], wbuf[:, :k], out=cbuf[:, :n], b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(cbuf[:, :n]).astype(np.float32), want)
    assert bool((cbuf[:, n:] == -1.0).all())
    # uniform operands against the oracle at the GEMM tolerance, the softcap epilogue on the same sums, and (fp32) a bias
    au, wu = synth.uniform(m + 23, (m, k)).astype(ndt), synth.uniform(n + 24, (n, k)).astype(ndt)
    ref = mm_want(oracle, au.astype(np.float32), wu.astype(np.float32).T)      # (the oracle and BLAS take the transposed view as it is)
    dau, dwu = dev(au), dev(wu)
    tol = TOL_F16_GEMM if half else TOL_F32
    got = host(ops.tensor_mm(dau, dwu, b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    assert scaled_rel_err(got, ref, math.sqrt(k) / 3.0) <= tol
    out = torch.empty((m, n), device="cuda", dtype=tdt)
    lib = capi.load()
    stream = torch.cuda.current_stream().cuda_stream
    name = "anygpu_gemm_f16_f32acc_softcap" if half else "anygpu_gemm_f32_softcap"
    capi.check(name, getattr(lib, name)(dau.data_ptr(), dwu.data_ptr(), out.data_ptr(), m, n, k, k, k, n, capi.B_COL_MAJOR, 2.0, stream))
    capped = oracle.softcap(ref, 2.0).reshape(m, n)
    # (the cap's slope is at most 1: a capped sum is off by no more than the sum, whose error grows with sqrt(k); the
    # outputs themselves stay within the cap)
    assert scaled_rel_err(host(out).astype(np.float32), capped, 2.0 / 3.0 if k <= 512 else 2.0) <= tol
    if not half:
        bias = synth.uniform(n + 25, (n,))
        dbias = dev(bias)
        capi.check("anygpu_gemm_f32", lib.anygpu_gemm_f32(dau.data_ptr(), dwu.data_ptr(), dbias.data_ptr(), out.data_ptr(), m, n, k,
                                                          k, k, n, capi.A_ROW_MAJOR, capi.B_COL_MAJOR, stream))
        assert scaled_rel_err(host(out), ref + bias[None, :], math.sqrt(k) / 3.0 + 1.0) <= tol


@pytest.mark.parametrize("layout", ["nk", "kn"])
@pytest.mark.parametrize("m,k,n", [(65, 2048, 14336), (80, 4096, 14336), (96, 2304, 9216), (130, 4096, 14336), (200, 2048, 8192)])
def test_mm_f32_rows_just_past_a_multiple_of_64(ops, oracle, layout, m, k, n):
    # products the launcher may divide by rows into the multiples of 64 and the rest (few-row kernels); entries -1 .. 1,
    # every sum exact in float32, so the result does not depend on whether it was divided; with a bias
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + 61, (m, k), -1, 1)
    b = synth.integers(n + 62, (k, n), -1, 1)
    bias = synth.integers(n + 63, (n,), -3, 3)
    want = mm_want(oracle, a, b) + bias[None, :].astype(np.float32)
    da, dbias = dev(a.astype(np.float32)), dev(bias.astype(np.float32))
    dw = dev(b.astype(np.float32)) if layout == "kn" else dev(np.ascontiguousarray(b.T).astype(np.float32))
    out = torch.empty((m, n), device="cuda")
    ldb = n if layout == "kn" else k
    capi.check("anygpu_gemm_f32", capi.load().anygpu_gemm_f32(
        da.data_ptr(), dw.data_ptr(), dbias.data_ptr(), out.data_ptr(), m, n, k, k, ldb, n, capi.A_ROW_MAJOR,
        capi.B_ROW_MAJOR if layout == "kn" else capi.B_COL_MAJOR, torch.cuda.current_stream().cuda_stream))
    assert np.array_equal(host(out), want)


ROUTING_EDGES = [
    # (rows, K in 128-byte steps of the dtype, columns): either side of what the launchers decide by
    (2, 2, 131072), (3, 2, 131072),                 # skinny kernels / band kernels
    (16, 3, 124672), (16, 3, 124416),               # 487 / 486 blocks of 256 columns: the wide band kernel or not
    (17, 2, 131072), (32, 1, 131072), (33, 2, 131072), (48, 2, 131072), (49, 2, 131072), (64, 3, 131072), (65, 2, 131072),
    (8, 2, 131328),                                 # 513 blocks: a third round with one block
    (8, 2, 131074), (8, 2, 131076),                 # columns no multiple of four / of eight
    (12, 5, 98304), (12, 4, 196608),                # 1.5 and 3 blocks per CU
    (128, 2, 32768), (129, 2, 32768), (128, 2, 32640),   # 128 x 128 tiles that fill the chip, or not quite
    (33, 4, 4096), (47, 4, 9216), (48, 4, 9216),    # fp32: band kernel / tiles first
    (257, 2, 14336), (384, 2, 14336), (385, 2, 14336), (300, 8, 8192),   # rows past a multiple of 256
]


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("m,steps,n", ROUTING_EDGES)
def test_mm_k_contiguous_weights_either_side_of_the_routing_rules(ops, oracle, dtype, m, steps, n):
    # small integers: every sum is exact, so whichever kernel a shape is routed to must return the oracle's result bit
    # for bit; the result sits inside a wider buffer whose other columns must stay untouched
    import torch
    from anygpu_amd import capi
    half = dtype == "f16"
    tdt, ndt = (torch.float16, np.float16) if half else (torch.float32, np.float32)
    k = steps * (64 if half else 32)
    a = synth.integers(m + 51, (m, k), -2, 2)
    w = synth.integers(n + 52, (n, k), -2, 2)
    want = mm_want(oracle, a, np.ascontiguousarray(w.T))
    assert np.abs(want).max() <= 2048
    cbuf = torch.full((m, n + 8), -3.0, device="cuda", dtype=tdt)
    ops.tensor_mm(dev(a.astype(ndt)), dev(w.astype(ndt)), out=cbuf[:, :n], b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(cbuf[:, :n]).astype(np.float32), want)
    assert bool((cbuf[:, n:] == -3.0).all())


@pytest.mark.parametrize("m,k,n", [(32, 128, 4096), (33, 128, 4096), (40, 256, 65536), (40, 256, 65540), (64, 96, 9216), (48, 64, 70000),
                                   (16, 2048, 2048), (17, 2048, 2048), (32, 2400, 2500), (24, 2464, 2500), (24, 4096, 1024)])
def test_mm_f32_n_contiguous_weights_either_side_of_the_routing_rules(ops, oracle, m, k, n):
    # [K, N] float32 weights: the band kernel for that layout up to 32 rows and for output heads, the tile kernels from 33
    # rows on up to 65536 columns (weights of up to 6 M elements: from 17 rows on); small integers, every sum exact
    a = synth.integers(m + 71, (m, k), -2, 2)
    b = synth.integers(n + 72, (k, n), -2, 2)
    want = mm_want(oracle, a, b)
    got = host(ops.tensor_mm(dev(a.astype(np.float32)), dev(b.astype(np.float32))))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("layout", ["nk", "kn"])
@pytest.mark.parametrize("m,k,n", [(16, 1023, 2048), (33, 1024, 2047), (5, 1028, 2052), (63, 2050, 1030), (1, 1025, 4100)])
def test_mm_f16_few_rows_of_operands_no_kernel_fetches_as_they_lie(ops, oracle, layout, m, k, n):
    # few rows, a K or an N that leaves the rows of an operand off 16-byte boundaries: where none of the kernels for few
    # rows takes the operands, aligned zero-padded copies are made and the product runs on those; small integers, exact
    from anygpu_amd import capi
    a = synth.integers(m + 61, (m, k), -2, 2)
    b = synth.integers(n + 62, (k, n), -2, 2)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da = dev(a.astype(np.float16))
    if layout == "kn":
        got = ops.tensor_mm(da, dev(b.astype(np.float16)))
    else:
        got = ops.tensor_mm(da, dev(np.ascontiguousarray(b.T).astype(np.float16)), b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(got).astype(np.float32), want)


@pytest.mark.parametrize("layout", ["nk", "kn"])
@pytest.mark.parametrize("m,k,n", [(16, 1023, 2048), (33, 1026, 2050), (100, 2050, 1030), (1, 1025, 4100), (127, 1031, 1100)])
def test_mm_f32_few_rows_of_operands_no_kernel_fetches_as_they_lie(ops, oracle, layout, m, k, n):
    # the same shapes in float32: a K that is no multiple of 4 (rows of A, and of [N, K] weights, off 16-byte boundaries)
    # goes to the general tile kernels (copies of 4-byte operands cost more than they save: 16 x 4098 -> 14338 110 -> 131 us)
    from anygpu_amd import capi
    a = synth.integers(m + 63, (m, k), -2, 2)
    b = synth.integers(n + 64, (k, n), -2, 2)
    want = mm_want(oracle, a, b)
    da = dev(a.astype(np.float32))
    if layout == "kn":
        got = ops.tensor_mm(da, dev(b.astype(np.float32)))
    else:
        got = ops.tensor_mm(da, dev(np.ascontiguousarray(b.T).astype(np.float32)), b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(got), want)
    # and with a bias, through the entry point that adds it
    bias = synth.integers(n + 65, (n,), -5, 5).astype(np.float32)
    w = dev(b.astype(np.float32)) if layout == "kn" else dev(np.ascontiguousarray(b.T).astype(np.float32))
    got = ops.tensor_gemm(da, w, dev(bias), b_layout=capi.B_ROW_MAJOR if layout == "kn" else capi.B_COL_MAJOR)
    assert np.array_equal(host(got), want + bias[None, :])


@pytest.mark.parametrize("layout", ["nk", "kn"])
@pytest.mark.parametrize("m,k,n", [(520, 4096, 14336), (264, 1024, 8192), (1100, 512, 9216), (640, 2048, 14336)])
def test_mm_f16_rows_just_past_a_multiple_of_256(ops, oracle, layout, m, k, n):
    # products the launcher may divide by rows into the whole multiples of 256 and the rest; small integers, every sum
    # exact, so the result does not depend on whether or where it was divided
    from anygpu_amd import capi
    a = synth.integers(m + 41, (m, k), -1, 1)
    b = synth.integers(n + 42, (k, n), -1, 1)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da = dev(a.astype(np.float16))
    if layout == "kn":
        got = ops.tensor_mm(da, dev(b.astype(np.float16)))
    else:
        got = ops.tensor_mm(da, dev(np.ascontiguousarray(b.T).astype(np.float16)), b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(got).astype(np.float32), want)


@pytest.mark.parametrize("layout", ["nk", "kn"])
@pytest.mark.parametrize("m,k,n", [(65, 128, 40000), (96, 192, 32768), (128, 64, 65536), (100, 256, 33000)])
def test_mm_f16_up_to_128_rows_against_many_columns(ops, oracle, layout, m, k, n):
    # 65 to 128 rows against weights with enough columns for 128 x 128 tiles to fill the chip: the four-wave kernel with
    # those tiles instead of half-empty 256 x 256 ones, both weight layouts; small integers, every sum exact
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + 31, (m, k), -2, 2)
    b = synth.integers(n + 32, (k, n), -2, 2)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da = dev(a.astype(np.float16))
    if layout == "kn":
        got = ops.tensor_mm(da, dev(b.astype(np.float16)))
    else:
        got = ops.tensor_mm(da, dev(np.ascontiguousarray(b.T).astype(np.float16)), b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(got).astype(np.float32), want)


@pytest.mark.parametrize("m,k,n", [(512, 256, 1003), (300, 512, 259), (128, 64, 65), (1000, 128, 4097), (65, 192, 7), (257, 320, 511)])
def test_mm_f16_k_contiguous_weights_result_rows_of_any_length(ops, oracle, m, k, n):
    # the tile kernels with [N, K] weights: N, the row length of C and its first element are free; integers, exact
    import torch
    from anygpu_amd import capi
    a = synth.integers(m + 5, (m, k), -2, 2)
    b = synth.integers(n + 6, (k, n), -2, 2)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da, dbt = dev(a.astype(np.float16)), dev(np.ascontiguousarray(b.T).astype(np.float16))
    assert np.array_equal(host(ops.tensor_mm(da, dbt, b_layout=capi.B_COL_MAJOR)).astype(np.float32), want)
    # C inside a wider buffer, starting one element in: nothing around it is touched
    cbuf = torch.full((m, n + 5), -1.0, device="cuda", dtype=torch.float16)
    ops.tensor_mm(da, dbt, out=cbuf[:, 1:n + 1], b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(cbuf[:, 1:n + 1]).astype(np.float32), want)
    assert bool((cbuf[:, :1] == -1.0).all()) and bool((cbuf[:, n + 1:] == -1.0).all())


@pytest.mark.parametrize("m,k,n", [(3, 64, 64), (4, 128, 72), (17, 136, 128), (64, 256, 64), (100, 320, 200), (5, 192, 1000),
                                   (3, 14336, 4096), (64, 4096, 1024), (256, 2048, 1024), (130, 8200, 512)])
def test_mm_f16_sparse_launches_of_small_tiles(ops, oracle, m, k, n):
    # few 64 x 64 tiles: the form with four LDS stages, from one slab (fewer slabs than stages) to hundreds, with a K
    # tail, and cut along K where the tiles alone leave CUs idle; both weight layouts; integers, so exact
    from anygpu_amd import capi
    a = synth.integers(m + 11, (m, k), -1, 1)
    b = synth.integers(n + 12, (k, n), -1, 1)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da = dev(a.astype(np.float16))
    dbt = dev(np.ascontiguousarray(b.T).astype(np.float16))
    assert np.array_equal(host(ops.tensor_mm(da, dbt, b_layout=capi.B_COL_MAJOR)).astype(np.float32), want)
    assert np.array_equal(host(ops.tensor_mm(da, dev(b.astype(np.float16)))).astype(np.float32), want)


@pytest.mark.parametrize("m,k,n", [(2048, 512, 4096), (2000, 576, 4000), (1024, 1032, 6100), (1024, 1032, 6144)])
def test_mm_f16_tiles_of_two_k_groups(ops, oracle, m, k, n):
    # shapes that take the 256 x 128 tile whose two wave groups split every slab and add up through LDS: whole and
    # ragged tiles, an odd number of slabs, a K tail; both weight layouts; integers, so exact
    from anygpu_amd import capi
    a = synth.integers(m + 21, (m, k), -1, 1)
    b = synth.integers(n + 22, (k, n), -1, 1)
    want = mm_want(oracle, a, b)
    assert np.abs(want).max() <= 2048
    da = dev(a.astype(np.float16))
    dbt = dev(np.ascontiguousarray(b.T).astype(np.float16))
    assert np.array_equal(host(ops.tensor_mm(da, dbt, b_layout=capi.B_COL_MAJOR)).astype(np.float32), want)
    if n % 8 == 0:
        assert np.array_equal(host(ops.tensor_mm(da, dev(b.astype(np.float16)))).astype(np.float32), want)


def test_mm_row_bands_integer_inputs_exact_streams_and_padded_buffers(ops, oracle):
    import torch
    from anygpu_amd import capi
    side = torch.cuda.Stream()
    for (m, k, n) in [(9, 256, 96), (16, 2048, 260), (32, 1024, 1000), (27, 4096, 36), (64, 4096, 132), (40, 512, 5000)]:
        a = synth.integers(1, (m, k), -4, 4)
        b = synth.integers(2, (k, n), -4, 4)
        bt = dev(np.ascontiguousarray(b.T))
        want = oracle.tensor_mm(a, b)
        assert np.array_equal(host(ops.tensor_mm(dev(a), bt, b_layout=capi.B_COL_MAJOR)), want)
        bias = synth.integers(3, (n,), -9, 9)
        assert np.array_equal(host(ops.tensor_gemm(dev(a), bt, dev(bias), b_layout=capi.B_COL_MAJOR)), oracle.tensor_gemm(a, b, bias))
        a16, b16 = a.astype(np.float16), np.ascontiguousarray(b.T).astype(np.float16)
        assert np.array_equal(host(ops.tensor_mm(dev(a16), dev(b16), b_layout=capi.B_COL_MAJOR)).astype(np.float32), want)
        # a second stream has a workspace of its own
        da = dev(a)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            got = ops.tensor_mm(da, bt, b_layout=capi.B_COL_MAJOR)
        side.synchronize()
        assert np.array_equal(host(got), want)
    # operands and result inside wider buffers
    abuf, bbuf = synth.uniform(4, (20, 200)), synth.uniform(5, (256, 300))
    cbuf = torch.full((20, 400), -1.0, device="cuda")
    ops.tensor_mm(dev(abuf)[:, :96], dev(bbuf)[:, :96], out=cbuf[:, :256], b_layout=capi.B_COL_MAJOR)
    got = host(cbuf)
    want = oracle.tensor_mm(np.ascontiguousarray(abuf[:, :96]), np.ascontiguousarray(bbuf[:, :96].T))
    assert scaled_rel_err(got[:, :256], want, math.sqrt(96) / 3.0) <= TOL_F32
    assert np.all(got[:, 256:] == -1.0)


@pytest.mark.parametrize("s", [1, 3, 8, 9, 16, 29, 50])
def test_gemm_epilogues_decode_step(ops, oracle, s):
    cap, hsize, vsize, isize = 30.0, 2304, 4000, 9216
    x = synth.normal(s, (1, s, hsize))
    w = synth.normal(2, (vsize, hsize)) * np.float32(0.3)
    got = host(ops.tensor_gemma_linear_softcap(dev(x), dev(w), cap))
    want = softcap_head_want(oracle, x, w, cap)
    assert scaled_rel_err(got, want, 0.3 * math.sqrt(hsize)) <= TOL_F32
    wg = synth.normal(3, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    wu = synth.normal(4, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    got = host(ops.mlp_gemma2_fused_upproj(dev(x), dev(wg), dev(wu)))
    want = upproj_want(oracle, x, wg, wu)
    assert scaled_rel_err(got, want, 1.0) <= TOL_F32


# fp16 products with the epilogues: the oracle's float32 operators on the fp16-rounded inputs, tolerance of the fp16 GEMM
F16_EPILOGUE_SHAPES = [
    # m, k, n: few rows (band kernels), one tile, ragged tiles of every size, a K tail, whole 256 tiles, several rounds
    (1, 2304, 1000), (16, 512, 520), (64, 256, 264), (100, 320, 200), (130, 64, 72), (300, 1000, 392), (513, 2304, 1160),
    (1024, 512, 2048), (2048, 192, 4096), (2304, 136, 4104),
    # k-contiguous weights in whole slabs: the four-wave kernels (128 x 128, 256 x 128 and 256 x 256 tiles, whole and ragged)
    (2048, 256, 2048), (2048, 128, 4096), (4096, 128, 4096), (1000, 192, 3000), (3000, 64, 4104),
    # few rows against a deep K (the plans cut along K, whose merge applies the epilogue), two rows (skinny kernels), so many
    # columns that the wide band kernel takes them, rows and columns a little past whole tiles (divided products)
    (8, 9216, 2304), (2, 4096, 2304), (5, 512, 131072), (48, 4096, 4096), (130, 4096, 2304), (300, 2048, 8192), (2048, 256, 10240),
]


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", F16_EPILOGUE_SHAPES)
def test_gemm_f16_bias(ops, oracle, layout, m, k, n):
    from anygpu_amd import capi
    a = synth.uniform(m + k, (m, k)).astype(np.float16)
    b = synth.uniform(k + n, (k, n)).astype(np.float16)
    bias = (synth.normal(n, (n,)) * np.float32(3.0)).astype(np.float16)
    want = gemm_want(oracle, oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(b), oracle.cvt_f16_to_f32(bias))
    if layout == "row":
        got = host(ops.tensor_gemm(dev(a), dev(b), dev(bias)))
    else:
        got = host(ops.tensor_gemm(dev(a), dev(np.ascontiguousarray(b.T)), dev(bias), b_layout=capi.B_COL_MAJOR))
    assert got.dtype == np.float16 and got.shape == (m, n)
    assert scaled_rel_err(got.astype(np.float32), want, math.sqrt(k) / 3.0 + 3.0) <= TOL_F16_GEMM
    # the bias is part of the result: without it the columns are off by it
    assert rel_l2(got.astype(np.float32) - oracle.cvt_f16_to_f32(bias)[None, :], mm_want(oracle, oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(b))) <= 2e-2


@pytest.mark.parametrize("m,k,n", F16_EPILOGUE_SHAPES)
def test_gemm_f16_softcap(ops, oracle, m, k, n):
    # the Gemma2 output head in fp16: weights [vocab, hidden], cap 30, logits well past the cap
    cap = 30.0
    x = synth.normal(m + k, (1, m, k)).astype(np.float16)
    w = (synth.normal(k + n, (n, k)) * np.float32(2.0)).astype(np.float16)
    got = host(ops.tensor_gemma_linear_softcap(dev(x), dev(w), cap)).astype(np.float32)
    want = softcap_head_want(oracle, oracle.cvt_f16_to_f32(x), oracle.cvt_f16_to_f32(w), cap)
    assert got.shape == (1, m, n)
    assert scaled_rel_err(got, want, min(cap, 2.0 * math.sqrt(k))) <= TOL_F16_GEMM
    assert np.all(np.abs(got) <= cap)


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("m,k,n", F16_EPILOGUE_SHAPES)
def test_gemm_f16_gelu_mul(ops, oracle, layout, m, k, n):
    # the Gemma2 MLP up-projection in fp16: gate and up weights side by side in one tile, A read once
    from anygpu_amd import capi
    x = synth.normal(m + k, (1, m, k)).astype(np.float16)
    wg = (synth.normal(n + 1, (k, n)) * np.float32(1.5 / math.sqrt(k))).astype(np.float16)
    wu = (synth.normal(n + 2, (k, n)) * np.float32(1.5 / math.sqrt(k))).astype(np.float16)
    want = upproj_want(oracle, oracle.cvt_f16_to_f32(x), oracle.cvt_f16_to_f32(wg), oracle.cvt_f16_to_f32(wu))
    if layout == "row":
        got = host(ops.mlp_gemma2_fused_upproj(dev(x), dev(wg), dev(wu))).astype(np.float32)
        swapped = host(ops.mlp_gemma2_fused_upproj(dev(x), dev(wu), dev(wg))).astype(np.float32)
    else:
        wgt, wut = dev(np.ascontiguousarray(wg.T)), dev(np.ascontiguousarray(wu.T))
        got = host(ops.mlp_gemma2_fused_upproj(dev(x), wgt, wut, b_layout=capi.B_COL_MAJOR)).astype(np.float32)
        swapped = host(ops.mlp_gemma2_fused_upproj(dev(x), wut, wgt, b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    assert got.shape == (1, m, n)
    assert scaled_rel_err(got, want, 1.5 * 1.5) <= TOL_F16_GEMM
    if n > 1:
        assert not np.allclose(swapped, got, atol=1e-2)       # the two weights are not interchangeable


def test_gemm_f16_epilogues_rejected_and_odd_shapes(ops, oracle):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    # K and N no multiples of 8: bias and softcap fall back to the plain product and a pass over it, the fused
    # up-projection has no kernel for such operands
    m, k, n = 70, 100, 51
    a = synth.uniform(1, (m, k)).astype(np.float16)
    b = synth.uniform(2, (k, n)).astype(np.float16)
    bias = synth.normal(3, (n,)).astype(np.float16)
    got = host(ops.tensor_gemm(dev(a), dev(b), dev(bias))).astype(np.float32)
    want = oracle.tensor_gemm(oracle.cvt_f16_to_f32(a), oracle.cvt_f16_to_f32(b), oracle.cvt_f16_to_f32(bias))
    assert scaled_rel_err(got, want, math.sqrt(k) / 3.0 + 1.0) <= TOL_F16_GEMM
    ad, bd = dev(a), dev(b)
    y = torch.full((m, n), 3.0, dtype=torch.float16, device="cuda")
    rc = lib.anygpu_gemm_f16_f32acc_gelu_mul(ad.data_ptr(), bd.data_ptr(), bd.data_ptr(), y.data_ptr(), m, n, k, k, n, n, capi.B_ROW_MAJOR, None)
    assert rc == capi.ANYGPU_ERR_UNSUPPORTED
    assert lib.anygpu_gemm_f16_f32acc_softcap(ad.data_ptr(), bd.data_ptr(), y.data_ptr(), m, n, k, k, n, n, capi.B_ROW_MAJOR, 0.0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert lib.anygpu_gemm_f16_f32acc_bias(ad.data_ptr(), bd.data_ptr(), None, y.data_ptr(), m, n, k, k, n, n, capi.B_ROW_MAJOR, None) == capi.ANYGPU_ERR_NULL_POINTER
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())


def _random_mm_shapes(seed, count, k_max):
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        regime = len(shapes) % 5
        if regime == 0:      # few rows, wide weights
            m, k, n = int(rng.integers(1, 70)), int(rng.integers(1, k_max)), int(rng.integers(1, 9000))
        elif regime == 1:    # few rows, deep K
            m, k, n = int(rng.integers(1, 70)), int(rng.integers(k_max // 2, k_max)), int(rng.integers(1, 700))
        elif regime == 2:    # a few tiles
            m, k, n = int(rng.integers(60, 600)), int(rng.integers(1, k_max)), int(rng.integers(60, 700))
        elif regime == 3:    # more than one round of big tiles
            m, k, n = int(rng.integers(1000, 2600)), int(rng.integers(1, 80)), int(rng.integers(3000, 6000))
        else:                # aligned versions of the above
            m, k, n = int(rng.integers(1, 40)) * 8, int(rng.integers(1, max(k_max // 64, 2))) * 64, int(rng.integers(1, 40)) * 128
        if m * k * n <= 400_000_000:
            shapes.append((m, k, n))
    return shapes


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_mm_random_shapes_integer_inputs_exact(ops, oracle, dtype):
    # small integers make every sum exact whatever the order, so every kernel family, every cut along K and every
    # division of a launch has to reproduce the oracle bit for bit; 40 shapes over the dispatch regimes, both layouts
    from anygpu_amd import capi
    k_max = 4000 if dtype == "f32" else 500          # |sum| < 2^24 in fp32; <= 2048, an fp16 integer, in half precision
    lo, hi = (-4, 4) if dtype == "f32" else (-2, 2)
    np_dt = np.float32 if dtype == "f32" else np.float16
    for i, (m, k, n) in enumerate(_random_mm_shapes(7 if dtype == "f32" else 8, 40, k_max)):
        a = synth.integers(100 + i, (m, k), lo, hi)
        b = synth.integers(200 + i, (k, n), lo, hi)
        want = mm_want(oracle, a, b)
        da = dev(a.astype(np_dt))
        got_row = host(ops.tensor_mm(da, dev(b.astype(np_dt)))).astype(np.float32)
        got_col = host(ops.tensor_mm(da, dev(np.ascontiguousarray(b.T).astype(np_dt)), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
        assert np.array_equal(got_row, want), ("row", m, k, n)
        assert np.array_equal(got_col, want), ("col", m, k, n)


def test_mm_empty_and_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    a = torch.zeros((4, 8), device="cuda", dtype=torch.float16)
    b = torch.zeros((8, 4), device="cuda", dtype=torch.float16)
    c = torch.full((4, 4), 3.0, device="cuda", dtype=torch.float16)
    f = lib.anygpu_gemm_f16_f32acc
    assert f(a.data_ptr(), b.data_ptr(), c.data_ptr(), 4, 4, 8, 4, 4, 4, 0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    assert f(a.data_ptr(), b.data_ptr(), c.data_ptr(), 4, 4, 8, 8, 4, 4, 7, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(a.data_ptr(), None, c.data_ptr(), 4, 4, 8, 8, 4, 4, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(a.data_ptr(), b.data_ptr(), c.data_ptr(), 4, -4, 8, 8, 4, 4, 0, None) == capi.ANYGPU_ERR_BAD_SHAPE
    assert f(a.data_ptr(), b.data_ptr(), c.data_ptr(), 0, 4, 8, 8, 4, 4, 0, None) == capi.ANYGPU_OK
    torch.cuda.synchronize()
    assert bool((c == 3.0).all())
    # K = 0: the product is all zeros
    z = ops.tensor_mm(torch.zeros((4, 0), device="cuda", dtype=torch.float32), torch.zeros((0, 5), device="cuda"))
    assert z.shape == (4, 5) and not bool(z.any())
    with pytest.raises(ValueError):
        ops.tensor_mm(torch.zeros((4, 8), device="cuda"), torch.zeros((7, 4), device="cuda"))


# =============================================================================================
# GEMM epilogues: Gemma2 output head (soft-capped logits), MLP gate / up projections
# =============================================================================================

@pytest.mark.parametrize("b,s,hsize,vsize", [(1, 1, 1, 1), (2, 9, 300, 1000), (1, 5, 64, 37), (1, 128, 256, 512),
                                             (3, 100, 130, 259), (1, 512, 512, 2048), (3, 100, 132, 260), (1, 50, 4100, 300)])
def test_gemma_linear_softcap_shapes(ops, oracle, b, s, hsize, vsize):
    cap = 30.0
    x = synth.normal(b * s + hsize, (b, s, hsize))
    w = synth.normal(vsize + hsize, (vsize, hsize)) * np.float32(4.0)      # logits reach well past the cap
    got = host(ops.tensor_gemma_linear_softcap(dev(x), dev(w), cap))
    want = softcap_head_want(oracle, x, w, cap)
    assert got.shape == (b, s, vsize)
    # |d softcap / d logit| <= 1: the GEMM's tolerance carries over, floored by the logit scale (at most the cap)
    assert scaled_rel_err(got, want, min(cap, 4.0 * math.sqrt(hsize))) <= TOL_F32
    assert np.all(np.abs(got) <= cap)


def test_gemma_linear_softcap_gemma2_hidden_2304_vocab_slice(ops, oracle):
    # srcs/models/gemma2/gemma_causallm.hpp:60-64: hidden 2304, cap 30; 32000 rows of the 256000-row table
    b, s, hsize, vsize, cap = 1, 96, 2304, 32000, 30.0
    x = synth.normal(1, (b, s, hsize))
    w = synth.normal(2, (vsize, hsize)) * np.float32(0.3)
    got = host(ops.tensor_gemma_linear_softcap(dev(x), dev(w), cap))
    idx = sample_rows(s, 12, seed=3)
    want = softcap_head_want(oracle, x[:, idx], w, cap)
    assert scaled_rel_err(got[:, idx], want, 0.3 * math.sqrt(hsize)) <= TOL_F32
    # all rows: tanh is odd and monotone, so atanh(y / cap) * cap recovers the logits; check their row sums
    logits = np.arctanh(np.clip(got.astype(np.float64) / cap, -1 + 1e-12, 1 - 1e-12)) * cap
    row_sum = x.astype(np.float64).reshape(s, hsize) @ w.astype(np.float64).sum(axis=0)
    assert np.max(np.abs(logits.reshape(s, vsize).sum(axis=1) - row_sum)) < 2e-3 * vsize


@pytest.mark.parametrize("b,s,hsize,isize", [(1, 1, 1, 1), (1, 37, 288, 1152), (1, 9, 2304, 1156), (2, 16, 520, 9216), (2, 5, 64, 37), (1, 128, 256, 512),
                                             (3, 50, 130, 259), (1, 256, 512, 2048), (3, 50, 132, 260),
                                             # 33 rows and more: two plain products and a combining pass (odd columns; large weights)
                                             (1, 70, 256, 259), (1, 33, 260, 512), (1, 300, 1024, 8192)])
def test_gemma_mlp_fused_upproj_shapes(ops, oracle, b, s, hsize, isize):
    x = synth.normal(b * s + hsize, (b, s, hsize))
    wg = synth.normal(isize + 1, (hsize, isize)) * np.float32(1.5 / math.sqrt(hsize))
    wu = synth.normal(isize + 2, (hsize, isize)) * np.float32(1.5 / math.sqrt(hsize))
    got = host(ops.mlp_gemma2_fused_upproj(dev(x), dev(wg), dev(wu)))
    want = upproj_want(oracle, x, wg, wu)
    assert got.shape == (b, s, isize)
    # gate and up are O(1.5) each; |gelu'| <= 1.13, so the product's error scale is that of the two sums
    assert scaled_rel_err(got, want, 1.5 * 1.5) <= TOL_F32
    # the two weights are not interchangeable
    if isize > 1:
        swapped = host(ops.mlp_gemma2_fused_upproj(dev(x), dev(wu), dev(wg)))
        assert not np.allclose(swapped, got, atol=1e-3)


def test_gemma_mlp_fused_upproj_gemma2_2304_9216(ops, oracle):
    # srcs/kernels/cuda/mlp_gemma2_fused_upproj.cuh:6-16: hidden 2304, intermediate 9216
    b, s, hsize, isize = 1, 256, 2304, 9216
    x = synth.normal(1, (b, s, hsize))
    wg = synth.normal(2, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    wu = synth.normal(3, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    got = host(ops.mlp_gemma2_fused_upproj(dev(x), dev(wg), dev(wu)))
    idx = sample_rows(s, 10, seed=4)
    want = upproj_want(oracle, x[:, idx], wg, wu)
    assert scaled_rel_err(got[:, idx], want, 1.0) <= TOL_F32
    # against the three-kernel chain on the device: same sums, so only the activation's rounding differs
    import torch
    g = ops.tensor_mm(dev(x.reshape(s, hsize)), dev(wg))
    u = ops.tensor_mm(dev(x.reshape(s, hsize)), dev(wu))
    chain = host(torch.nn.functional.gelu(g, approximate="tanh") * u)
    assert scaled_rel_err(got.reshape(s, isize), chain, 1.0) <= TOL_F32


@pytest.mark.parametrize("m,hsize,isize", [(3, 288, 1152), (12, 288, 1152), (32, 2304, 516), (17, 64, 40), (64, 4608, 300), (37, 2304, 9216),
                                           # two products (priced) / the fused four-wave kernel in whole rounds / ragged columns
                                           (100, 512, 1030), (300, 2304, 9216), (384, 2304, 9216)])
def test_gemm_gelu_mul_k_contiguous_weights(ops, oracle, m, hsize, isize):
    # the fused up-projection with the weights stored [intermediate, hidden], through the C entry point
    import torch
    from anygpu_amd import capi
    x = synth.normal(m, (m, hsize))
    wg = synth.normal(3, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    wu = synth.normal(4, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    want = upproj_want(oracle, x, wg, wu)
    dx, dg, du = dev(x), dev(np.ascontiguousarray(wg.T)), dev(np.ascontiguousarray(wu.T))
    out = torch.empty((m, isize), device="cuda")
    rc = capi.load().anygpu_gemm_f32_gelu_mul(dx.data_ptr(), dg.data_ptr(), du.data_ptr(), out.data_ptr(), m, isize, hsize,
                                              hsize, hsize, isize, capi.B_COL_MAJOR, None)
    assert rc == capi.ANYGPU_OK
    assert scaled_rel_err(host(out), want, 1.0) <= TOL_F32


def test_gemm_gelu_mul_as_two_products_whose_operands_want_copies(ops, oracle):
    # 200 rows: the fused up-projection runs as two plain products into planes of the stream's workspace.  K is no
    # multiple of 32, so each product would like aligned zero-padded copies of its operands, 80 MB for these weights:
    # more than the library's buffer holds behind the planes, and the buffer must not grow (be freed and allocated
    # anew) while the planes live in it.  Twice, so that a buffer that did change hands shows.
    import torch
    from anygpu_amd import capi
    m, hsize, isize = 200, 2052, 9216
    x = synth.normal(m, (m, hsize))
    wg = synth.normal(5, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    wu = synth.normal(6, (hsize, isize)) * np.float32(1.0 / math.sqrt(hsize))
    want = upproj_want(oracle, x, wg, wu)
    dx, dg, du = dev(x), dev(np.ascontiguousarray(wg.T)), dev(np.ascontiguousarray(wu.T))
    for _ in range(2):
        out = torch.empty((m, isize), device="cuda")
        rc = capi.load().anygpu_gemm_f32_gelu_mul(dx.data_ptr(), dg.data_ptr(), du.data_ptr(), out.data_ptr(), m, isize, hsize,
                                                  hsize, hsize, isize, capi.B_COL_MAJOR, None)
        assert rc == capi.ANYGPU_OK
        assert scaled_rel_err(host(out), want, 1.0) <= TOL_F32
    # and the plain product of the same operands afterwards (which may now grow the buffer for its copies)
    got = host(ops.tensor_mm(dx, dg, b_layout=capi.B_COL_MAJOR))
    assert scaled_rel_err(got, mm_want(oracle, x, wg), 1.0) <= TOL_F32


def test_gemm_epilogues_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    a = torch.zeros((4, 8), device="cuda")
    w = torch.zeros((8, 4), device="cuda")
    c = torch.full((4, 4), 3.0, device="cuda")
    f = lib.anygpu_gemm_f32_softcap
    assert f(a.data_ptr(), w.data_ptr(), c.data_ptr(), 4, 4, 8, 8, 4, 4, capi.B_ROW_MAJOR, 0.0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(a.data_ptr(), w.data_ptr(), c.data_ptr(), 4, 4, 8, 8, 4, 4, capi.B_ROW_MAJOR, float("nan"), None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(a.data_ptr(), w.data_ptr(), c.data_ptr(), 4, 4, 8, 8, 2, 4, capi.B_ROW_MAJOR, 30.0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    g = lib.anygpu_gemm_f32_gelu_mul
    assert g(a.data_ptr(), w.data_ptr(), None, c.data_ptr(), 4, 4, 8, 8, 4, 4, capi.B_ROW_MAJOR, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert g(a.data_ptr(), w.data_ptr(), w.data_ptr(), c.data_ptr(), 4, 0, 8, 8, 4, 4, capi.B_ROW_MAJOR, None) == capi.ANYGPU_OK
    torch.cuda.synchronize()
    assert bool((c == 3.0).all())
    with pytest.raises(ValueError):
        ops.tensor_gemma_linear_softcap(torch.zeros((1, 4, 8), device="cuda"), torch.zeros((5, 7), device="cuda"), 30.0)


# =============================================================================================
# the caller of the path: masked, scaled dot-product attention
# =============================================================================================

@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("batch,m,k,n", [(1, 64, 64, 64), (5, 16, 128, 16), (32, 256, 64, 256), (3, 100, 37, 60), (8, 128, 256, 64),
                                         (2, 129, 100, 131), (3, 128, 4096, 128), (2, 300, 1001, 257),
                                         (2, 1000, 520, 4096)])     # (the last: fp16 takes the 256 x 128 tile in two k groups)
def test_mm_batched(ops, oracle, dtype, batch, m, k, n):
    from anygpu_amd import capi
    np_dt = np.float16 if dtype == "f16" else np.float32
    a = synth.uniform(batch + m, (batch, m, k)).astype(np_dt)
    bt = synth.uniform(batch + n, (batch, n, k)).astype(np_dt)
    a32 = oracle.cvt_f16_to_f32(a) if dtype == "f16" else a
    b32 = oracle.cvt_f16_to_f32(bt) if dtype == "f16" else bt
    want = np.stack([oracle.tensor_mm(a32[i], b32[i].T) for i in range(batch)])
    tol = TOL_F16_GEMM if dtype == "f16" else TOL_F32
    got_nt = host(ops.tensor_mm_batched(dev(a), dev(bt), b_layout=capi.B_COL_MAJOR)).astype(np.float32)
    assert scaled_rel_err(got_nt, want, math.sqrt(k) / 3.0) <= tol
    got_nn = host(ops.tensor_mm_batched(dev(a), dev(np.ascontiguousarray(bt.transpose(0, 2, 1))))).astype(np.float32)
    assert scaled_rel_err(got_nn, want, math.sqrt(k) / 3.0) <= tol


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("rows,cols,q_len,cap", [(64, 64, 64, 0.0), (96, 48, 48, 0.0), (40, 72, 40, 30.0), (33, 100, 33, 0.0),
                                                 (256, 2048, 128, 0.0), (12, 8192, 4, 50.0),
                                                 # several heads over one mask, query counts that do not fill the blocks' row
                                                 # groups (sixteen rows, four rows, one row per block); rows walked twice,
                                                 # whole and at odd widths
                                                 (3 * 37, 40, 37, 0.0), (5 * 9, 600, 9, 0.0), (20 * 70, 1024, 70, 30.0), (6 * 7, 20000, 7, 0.0),
                                                 (4 * 16, 40000, 16, 0.0), (2 * 3, 70001, 3, 50.0), (10, 33000, 10, 0.0)])
def test_softmax_with_mask_tensor(ops, oracle, dtype, rows, cols, q_len, cap):
    # the mask arrives as data (the reference's attention interface); it must agree with the index-rule form
    np_dt = np.float16 if dtype == "f16" else np.float32
    alpha = 0.125
    x = synth.normal(rows + cols, (rows, cols), std=8.0).astype(np_dt)
    diag = cols - q_len
    mask = oracle.slide_mask(oracle.causal_mask(q_len, cols, diag=diag), max(cols // 3, 1)) if rows != 33 \
        else oracle.causal_mask(q_len, cols, diag=diag)
    with np.errstate(over="ignore"):
        mask_dev = mask.astype(np_dt)       # float lowest becomes -inf in half precision: masked all the same
    got = host(ops.tensor_softmax_masked(dev(x), dev(mask_dev), alpha=alpha, softcap=cap, q_len=q_len)).astype(np.float32)
    x32 = oracle.cvt_f16_to_f32(x) if dtype == "f16" else x
    s = oracle.tensor_mul_scalar(x32, alpha).reshape(rows, cols)
    if cap:
        s = oracle.softcap(s, cap).reshape(rows, cols)
    m32 = np.tile(mask.astype(np.float32), (rows // q_len, 1))
    want = oracle.tensor_softmax(oracle.tensor_add(s, m32))
    tol = TOL_F16_ROWOPS if dtype == "f16" else TOL_F32
    assert np.all(got[m32 != 0] == 0.0)
    assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= tol


def test_sdp_attention_masked_scaled_fwd(ops, oracle):
    import torch
    # the reference's golden shape [1, 32, 16, 128] with a tril -inf mask and scale 0.125, float32
    q, k, v = (synth.normal(s, (1, 32, 16, 128)) for s in (1, 2, 3))
    mask = oracle.causal_mask(16, 16).reshape(1, 1, 16, 16)
    want = oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask, 0.125, threads=8)
    got = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask), 0.125))
    ok, worst = oracle.compare_data_buffers(got, want)            # the reference's gate: abs 1e-3
    assert ok, worst
    assert scaled_rel_err(got, want, 1.0) <= TOL_F32
    # a Gemma2-like block in half precision: 8 heads, 512 queries and keys, d = 256, causal + window 128
    h, n, d = 8, 512, 256
    q, k, v = (synth.normal(s, (1, h, n, d)).astype(np.float16) for s in (4, 5, 6))
    mask = oracle.slide_mask(oracle.causal_mask(n, n), 128).reshape(1, 1, n, n)
    want = oracle.sdp_attention_masked_scaled_fwd(*(oracle.cvt_f16_to_f32(t) for t in (q, k, v)), mask, 0.0625, threads=8)
    with np.errstate(over="ignore"):
        mask16 = mask.astype(np.float16)
    got = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask16), 0.0625)).astype(np.float32)
    assert rel_l2(got, want) <= 1e-2
    assert scaled_rel_err(got, want, 1.0) <= TOL_F16_GEMM


@pytest.mark.parametrize("heads,n_q,n_k,d,kind", [
    (4, 100, 100, 64, "causal"), (2, 130, 131, 128, "slide"), (3, 257, 257, 256, "slide"), (2, 64, 203, 128, "random"),
    (2, 33, 1001, 256, "random"), (8, 200, 5000, 64, "causal"),          # (the last: few query blocks, the key range in parts)
    (2, 70, 70, 128, "blind_rows"), (1, 17, 3, 64, "random"),
    # key ranges hidden from whole blocks of queries (key tiles the visible-tile map of the mask leaves out), ragged last tiles and blocks
    (2, 300, 1500, 128, "slide"), (3, 200, 2100, 64, "stripes"), (2, 150, 4200, 256, "stripes"), (1, 520, 1030, 128, "stripes"),
])
def test_sdp_attention_fused_kernel_f32_with_mask_tensor(ops, oracle, monkeypatch, heads, n_q, n_k, d, kind):
    # the reference's own attention interface (srcs/transformers/sdp.hpp:207-274): the mask arrives as a tensor.  In
    # float32 one kernel reads it as data; against the oracle's operator chain and against the three-launch form
    # (batched product, softmax with the mask tensor, batched product) on the device.
    import torch
    q = synth.normal(1 + n_q, (1, heads, n_q, d))
    k = synth.normal(2 + n_k, (1, heads, n_k, d))
    v = synth.normal(3 + d, (1, heads, n_k, d))
    alpha = float(d) ** -0.5
    diag = n_k - n_q
    if kind == "causal":
        mask = oracle.causal_mask(n_q, n_k, diag=diag)
    elif kind == "slide":
        mask = oracle.slide_mask(oracle.causal_mask(n_q, n_k, diag=diag), max(n_k // 3, 1))
    else:
        # finite biases everywhere, a third of the keys hidden at random (every query keeps key 0)
        rng = np.random.default_rng(n_q * 1000 + n_k)
        mask = rng.normal(0.0, 2.0, (n_q, n_k)).astype(np.float32)
        mask[rng.random((n_q, n_k)) < 0.33] = -np.inf
        mask[:, 0] = 0.5
        if kind == "stripes":
            hide_key_stripes(mask, rng)
        if kind == "blind_rows":
            mask[5] = -np.inf                     # queries without a visible key: zeros, where the operator chain has NaN
            mask[n_q // 2] = -np.inf
            mask[n_q - 1, 1:] = np.finfo(np.float32).min      # the float lowest of the reference's mask builders hides as well
    mask4 = np.ascontiguousarray(mask, dtype=np.float32).reshape(1, 1, n_q, n_k)
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask4, alpha, threads=8)
    # with the visible-tile map of the mask (a pass over the mask ahead of the kernel; by default only for large masks)
    # and without
    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", "0")
    got = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask4), alpha))
    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", str(1 << 60))
    without_map = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask4), alpha))
    # (few query blocks go out in parts of their key range, cut by visible tiles with the map and by range without:
    # another order of summation)
    assert scaled_rel_err(got, without_map, 1.0) <= 1e-5
    assert got.shape == q.shape and got.dtype == np.float32 and np.isfinite(got).all()
    blind = ~np.isfinite(want).all(axis=-1)
    assert blind.sum() == (2 * heads if kind == "blind_rows" else 0)
    assert not got[blind].any()
    assert scaled_rel_err(got[~blind], want[~blind], 1.0) <= TOL_F32
    # the three launches on the device
    scores = ops.tensor_mm_batched(dev(q[0]), dev(k[0]), b_layout=__import__("anygpu_amd").capi.B_COL_MAJOR)
    probs = ops.tensor_softmax_masked(scores.reshape(-1, n_k), dev(mask4.reshape(n_q, n_k)), alpha=alpha, q_len=n_q)
    three = host(ops.tensor_mm_batched(probs.reshape(heads, n_q, n_k), dev(v[0])))
    assert scaled_rel_err(got[0][~blind[0]], three[~blind[0]], 1.0) <= TOL_F32 * 2
    # the C entry point's own checks
    from anygpu_amd import capi
    f = capi.load().anygpu_sdp_attention_fwd_masked_f32
    dq, dk, dv, dm = dev(q), dev(k), dev(v), dev(mask4)
    y = torch.full(q.shape, 3.0, device="cuda")
    assert f(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), None, y.data_ptr(), heads, 1, n_q, n_k, d, n_k, alpha, 0.0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dm.data_ptr(), y.data_ptr(), heads, 1, n_q, n_k, d, n_k - 1, alpha, 0.0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())


@pytest.mark.parametrize("heads,n_q,n_k,d,kind", [
    (4, 100, 100, 64, "causal"), (2, 130, 131, 128, "slide"), (3, 257, 257, 256, "slide"), (2, 64, 203, 128, "random"),
    (2, 33, 1001, 256, "random"), (8, 200, 5000, 64, "causal"),          # (the last: few query blocks, the key range in parts)
    (2, 70, 70, 128, "blind_rows"), (1, 17, 3, 64, "random"), (2, 300, 300, 256, "odd_stride"),
    # key ranges hidden from whole blocks of queries (key tiles the visible-tile map of the mask leaves out), ragged last tiles and blocks
    (2, 300, 1500, 128, "slide"), (3, 200, 2100, 64, "stripes"), (2, 150, 4200, 256, "stripes"), (1, 520, 1030, 128, "stripes"),
    (2, 260, 1500, 64, "odd_stride"),
])
def test_sdp_attention_fused_kernel_f16_with_mask_tensor(ops, oracle, monkeypatch, heads, n_q, n_k, d, kind):
    # the same interface in half precision: one kernel reads the mask (halves, -inf where a key is hidden) as data;
    # against the oracle's operator chain on the up-cast operands and against the three launches on the device
    import torch
    from anygpu_amd import capi
    q = synth.normal(1 + n_q, (1, heads, n_q, d)).astype(np.float16)
    k = synth.normal(2 + n_k, (1, heads, n_k, d)).astype(np.float16)
    v = synth.normal(3 + d, (1, heads, n_k, d)).astype(np.float16)
    alpha = float(d) ** -0.5
    diag = n_k - n_q
    if kind == "causal":
        mask = oracle.causal_mask(n_q, n_k, diag=diag)
    elif kind in ("slide", "odd_stride"):
        mask = oracle.slide_mask(oracle.causal_mask(n_q, n_k, diag=diag), max(n_k // 3, 1))
    else:
        rng = np.random.default_rng(n_q * 1000 + n_k)
        mask = rng.normal(0.0, 2.0, (n_q, n_k)).astype(np.float32)
        mask[rng.random((n_q, n_k)) < 0.33] = -np.inf
        mask[:, 0] = 0.5
        if kind == "stripes":
            hide_key_stripes(mask, rng)
        if kind == "blind_rows":
            mask[5] = -np.inf                     # queries without a visible key: zeros, where the operator chain has NaN
            mask[n_q // 2] = -np.inf
    with np.errstate(over="ignore"):
        mask16 = np.ascontiguousarray(mask, dtype=np.float32).astype(np.float16).reshape(1, 1, n_q, n_k)
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle.sdp_attention_masked_scaled_fwd(*(oracle.cvt_f16_to_f32(t) for t in (q, k, v)), mask16.astype(np.float32), alpha, threads=8)
    dq, dk, dv, dm = dev(q), dev(k), dev(v), dev(mask16)
    if kind == "odd_stride":
        # mask rows an odd number of halves apart, starting off a 4-byte boundary, through the C entry point itself
        pitch = n_k + 3
        store = torch.full((n_q * pitch + 1,), float("nan"), dtype=torch.float16, device="cuda")
        rows = store[1:].reshape(n_q, pitch)
        rows[:, :n_k] = dm.reshape(n_q, n_k)

        def run():
            y = torch.empty_like(dq)
            rc = capi.load().anygpu_sdp_attention_fwd_masked_f16(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), rows.data_ptr(), y.data_ptr(),
                                                                 heads, 1, n_q, n_k, d, pitch, alpha, 0.0, None)
            assert rc == capi.ANYGPU_OK
            return host(y).astype(np.float32)
    else:
        def run():
            return host(ops.sdp_attention_masked_scaled_fwd(dq, dk, dv, dm, alpha)).astype(np.float32)
    # with the visible-tile map of the mask (a pass over the mask ahead of the kernel; by default only for large masks)
    # and without (few query blocks go out in parts of their key range, cut by visible tiles with the map and by range
    # without: another order of summation, a last place of the half result)
    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", "0")
    got = run()
    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", str(1 << 60))
    assert scaled_rel_err(got, run(), 1.0) <= TOL_F16_ROWOPS
    assert got.shape == q.shape and np.isfinite(got).all()
    blind = ~np.isfinite(want).all(axis=-1)
    assert blind.sum() == (2 * heads if kind == "blind_rows" else 0)
    assert not got[blind].any()
    assert rel_l2(got[~blind], want[~blind]) <= 1e-2
    assert scaled_rel_err(got[~blind], want[~blind], 1.0) <= TOL_F16_GEMM
    # the three launches on the device
    scores = ops.tensor_mm_batched(dq[0], dk[0], b_layout=capi.B_COL_MAJOR)
    probs = ops.tensor_softmax_masked(scores.reshape(-1, n_k), dm.reshape(n_q, n_k), alpha=alpha, q_len=n_q)
    three = host(ops.tensor_mm_batched(probs.reshape(heads, n_q, n_k), dv[0])).astype(np.float32)
    assert scaled_rel_err(got[0][~blind[0]], three[~blind[0]], 1.0) <= TOL_F16_GEMM
    # the C entry point's own checks
    f = capi.load().anygpu_sdp_attention_fwd_masked_f16
    y = torch.full(q.shape, 3.0, device="cuda", dtype=torch.float16)
    assert f(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), None, y.data_ptr(), heads, 1, n_q, n_k, d, n_k, alpha, 0.0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dm.data_ptr(), y.data_ptr(), heads, 1, n_q, n_k, d, n_k - 1, alpha, 0.0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    assert f(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dm.data_ptr() + 1, y.data_ptr(), heads, 1, n_q, n_k, d, n_k, alpha, 0.0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())


def test_sdp_attention_f32_mask_tensor_blocks_in_two_parts_of_their_visible_tiles(ops, oracle, monkeypatch):
    # as many query blocks as one to four rounds of the chip (16 heads x 18 blocks of 64 queries): with the map of the mask
    # every block goes out in two parts, each with half of its visible tiles, and a merge launch; against the run without
    # the map (whole blocks), against the three launches on the device, and two of the heads against the oracle
    import torch
    from anygpu_amd import capi
    heads, n_q, n_k, d = 16, 1100, 2100, 64
    q = synth.normal(71, (1, heads, n_q, d))
    k = synth.normal(72, (1, heads, n_k, d))
    v = synth.normal(73, (1, heads, n_k, d))
    alpha = float(d) ** -0.5
    rng = np.random.default_rng(74)
    mask = rng.normal(0.0, 1.0, (n_q, n_k)).astype(np.float32)
    hide_key_stripes(mask, rng)
    mask4 = mask.reshape(1, 1, n_q, n_k)
    dq, dk, dv, dm = dev(q), dev(k), dev(v), dev(mask4)
    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", "0")
    got = host(ops.sdp_attention_masked_scaled_fwd(dq, dk, dv, dm, alpha))
    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", str(1 << 60))
    whole = host(ops.sdp_attention_masked_scaled_fwd(dq, dk, dv, dm, alpha))
    assert np.isfinite(got).all()
    assert scaled_rel_err(got, whole, 1.0) <= 1e-5
    assert not np.array_equal(got, whole), "the two runs were expected to sum in different orders"
    scores = ops.tensor_mm_batched(dq[0], dk[0], b_layout=capi.B_COL_MAJOR)
    probs = ops.tensor_softmax_masked(scores.reshape(-1, n_k), dm.reshape(n_q, n_k), alpha=alpha, q_len=n_q)
    three = host(ops.tensor_mm_batched(probs.reshape(heads, n_q, n_k), dv[0]))
    assert scaled_rel_err(got[0], three, 1.0) <= TOL_F32 * 2
    for h in (0, heads - 1):
        want = oracle.sdp_attention_masked_scaled_fwd(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], mask4, alpha, threads=8)
        assert scaled_rel_err(got[:, h:h + 1], want, 1.0) <= TOL_F32


ATTN_CASES = [
    # heads, kv_heads, n_q, n_k, d, alpha, softcap, causal, window
    (2, 2, 16, 16, 64, 0.125, 0.0, False, 0),
    (3, 3, 100, 100, 64, 0.125, 0.0, True, 0),
    (4, 2, 130, 130, 128, 0.0884, 0.0, True, 0),
    (2, 1, 257, 257, 256, 0.0625, 50.0, True, 96),
    (2, 2, 64, 200, 128, 0.0884, 0.0, True, 0),          # queries are the last 64 positions of a 200-key cache
    (2, 2, 1, 300, 128, 0.0884, 30.0, True, 128),        # decode step
    (1, 1, 200, 77, 64, 0.125, 0.0, False, 0),
    (2, 2, 192, 192, 64, 0.125, 0.0, False, 40),         # window without the causal rule
    # a chunk of a long prompt against its cache: few query blocks, long key ranges, every block in several parts
    (8, 1, 200, 5000, 64, 0.125, 0.0, True, 0),
    (4, 2, 130, 3000, 128, 0.0884, 30.0, True, 1000),
    (2, 2, 300, 2500, 128, 0.0884, 0.0, False, 0),
]


@pytest.mark.parametrize("case", ATTN_CASES)
def test_sdp_attention_fused_kernel(ops, oracle, case):
    heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window = case
    q = synth.normal(1 + n_q, (1, heads, n_q, d)).astype(np.float16)
    k = synth.normal(2 + n_k, (1, kv_heads, n_k, d)).astype(np.float16)
    v = synth.normal(3 + d, (1, kv_heads, n_k, d)).astype(np.float16)
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window)).astype(np.float32)
    want = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t)[0] for t in (q, k, v)), alpha=alpha, softcap=cap,
                                      causal=causal, window=window, q_per_kv=heads // kv_heads, threads=8)
    assert got.shape == (1, heads, n_q, d)
    # outputs are convex combinations of N(0, 1) values: scale floor 1
    assert scaled_rel_err(got[0], want, 1.0) <= TOL_F16_ROWOPS * 2          # p is rounded to fp16 before the second product
    assert rel_l2(got[0], want) <= 2e-3


def _random_attention_cases(count, seed):
    import random
    rnd = random.Random(seed)
    cases = []
    for _ in range(count):
        d = rnd.choice([64, 128, 256])
        kv_heads = rnd.choice([1, 2, 3])
        group = rnd.choice([1, 2, 4, 8])
        n_q = rnd.choice([1, 17, 64, 100, 129, 300, 512, 777])
        n_k = n_q + rnd.choice([0, 0, 5, 64, 200])
        causal = rnd.choice([True, True, False])
        window = rnd.choice([0, 0, 33, 128, 500]) if causal else 0
        cap = rnd.choice([0.0, 0.0, 30.0])
        alpha = rnd.choice([d ** -0.5, 0.0625, -0.05])
        cases.append((kv_heads * group, kv_heads, n_q, n_k, d, alpha, cap, causal, window))
    return cases


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_sdp_attention_fused_kernel_random_shapes(ops, oracle, dtype):
    # many (heads, groups, lengths, masks) at random: every (head, query block) of the one-dimensional grid's block
    # walk has to turn up exactly once, on both tile paths of the fp16 kernel (softcap or not at head dimension 256)
    for case in _random_attention_cases(24, 7 if dtype == "f16" else 8):
        heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window = case
        np_t = np.float16 if dtype == "f16" else np.float32
        q = synth.normal(1 + n_q, (1, heads, n_q, d)).astype(np_t)
        k = synth.normal(2 + n_k, (1, kv_heads, n_k, d)).astype(np_t)
        v = synth.normal(3 + d, (1, kv_heads, n_k, d)).astype(np_t)
        got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window)).astype(np.float32)
        want = oracle.sdp_attention_rules(*(t.astype(np.float32)[0] for t in (q, k, v)), alpha=alpha, softcap=cap,
                                          causal=causal, window=window, q_per_kv=heads // kv_heads, threads=8)
        tol = TOL_F16_ROWOPS * 2 if dtype == "f16" else TOL_F32 * 2
        assert scaled_rel_err(got[0], want, 1.0) <= tol, case


# head_dim 256 runs the kernel that takes S of tile t + 1 beside the softmax of tile t: tile counts of
# one and two (the pipelined loop body not entered / entered once), a last tile that is not whole, a key range longer
# than the queries, windows below a tile and without the causal rule, queries without a visible key, grouped heads
ATTN_D256_CASES = [
    (2, 2, 17, 63, 256, 0.0625, 50.0, True, 0),
    (2, 2, 17, 64, 256, 0.0625, 50.0, True, 0),
    (2, 2, 20, 65, 256, 0.0625, 50.0, False, 0),
    (2, 1, 128, 128, 256, 0.0625, 30.0, True, 0),
    (2, 1, 129, 129, 256, 0.0625, 30.0, True, 0),
    (4, 2, 200, 333, 256, 0.0625, 50.0, True, 0),
    (2, 2, 300, 300, 256, -0.05, 50.0, True, 33),
    (2, 2, 260, 260, 256, 0.0625, 50.0, False, 70),
    (2, 2, 100, 40, 256, 0.0625, 50.0, True, 0),
    (8, 2, 640, 700, 256, 0.0625, 50.0, True, 200),
    # the same kernel without softcap
    (2, 2, 17, 65, 256, 0.0625, 0.0, True, 0),
    (2, 1, 129, 129, 256, 0.0625, 0.0, True, 0),
    (4, 2, 200, 333, 256, -0.05, 0.0, True, 33),
    (2, 2, 260, 260, 256, 0.0625, 0.0, False, 70),
    (2, 2, 100, 40, 256, 0.0625, 0.0, True, 0),
    # few query blocks against a long cache: every block in several parts of its key range
    (4, 1, 150, 4100, 256, 0.0625, 50.0, True, 0),
    (2, 2, 129, 2000, 256, 0.0625, 0.0, True, 700),
]


@pytest.mark.parametrize("case", ATTN_D256_CASES)
def test_sdp_attention_fused_kernel_head_dim_256(ops, oracle, case):
    heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window = case
    q = synth.normal(1 + n_q, (1, heads, n_q, d)).astype(np.float16)
    k = synth.normal(2 + n_k, (1, kv_heads, n_k, d)).astype(np.float16)
    v = synth.normal(3 + d, (1, kv_heads, n_k, d)).astype(np.float16)
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window)).astype(np.float32)
    want = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t)[0] for t in (q, k, v)), alpha=alpha, softcap=cap,
                                      causal=causal, window=window, q_per_kv=heads // kv_heads, threads=8)
    assert got.shape == (1, heads, n_q, d)
    blind = ~np.isfinite(want).all(axis=-1)                      # queries without a visible key: zeros
    assert not got[0][blind].any()
    assert np.isfinite(got).all()
    assert scaled_rel_err(got[0][~blind], want[~blind], 1.0) <= TOL_F16_ROWOPS * 2, case


@pytest.mark.parametrize("case", ATTN_CASES)
def test_sdp_attention_fused_kernel_f32(ops, oracle, case):
    # the float32 form of the same kernel: fp32 operands and the fp32 matrix instruction, fp32 tolerance
    heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window = case
    q = synth.normal(1 + n_q, (1, heads, n_q, d))
    k = synth.normal(2 + n_k, (1, kv_heads, n_k, d))
    v = synth.normal(3 + d, (1, kv_heads, n_k, d))
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window))
    want = oracle.sdp_attention_rules(q[0], k[0], v[0], alpha=alpha, softcap=cap, causal=causal, window=window,
                                      q_per_kv=heads // kv_heads, threads=8)
    assert got.shape == (1, heads, n_q, d) and got.dtype == np.float32
    blind = ~np.isfinite(want).all(axis=-1)                      # queries without a visible key: zeros
    assert not got[0][blind].any()
    assert scaled_rel_err(got[0][~blind], want[~blind], 1.0) <= TOL_F32


def test_sdp_attention_fused_kernel_f32_structure(ops, oracle):
    heads, n, d = 2, 160, 128
    q, k, v = (synth.normal(s, (heads, n, d)) for s in (1, 2, 3))
    y = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0884, causal=True))
    assert np.array_equal(y[:, 0, :], v[:, 0, :])               # first causal row attends to key 0 only
    k2, v2 = k.copy(), v.copy()
    k2[:, 100:, :] += 1.0
    v2[:, 100:, :] -= 2.0
    y2 = host(ops.sdp_attention_fwd(dev(q), dev(k2), dev(v2), 0.0884, causal=True))
    assert np.array_equal(y[:, :100, :], y2[:, :100, :])         # causality, bit for bit
    assert not np.array_equal(y[:, 100:, :], y2[:, 100:, :])
    ys = host(ops.sdp_attention_fwd(dev(q), dev(k[:, :60]), dev(v[:, :60]), 0.0884, causal=True))
    assert not ys[:, :100, :].any() and ys[:, 100:, :].any()
    # against the three-launch form with the mask as data
    mask = oracle.slide_mask(oracle.causal_mask(n, n), 48).reshape(1, n, n)
    three = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask), 0.0884))
    fused = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0884, causal=True, window=48))
    assert scaled_rel_err(fused, three, 1.0) <= TOL_F32
    # integer-valued v and a single visible key per query (window 1): the output is that row of v exactly
    vi = synth.integers(5, (heads, n, d), -8, 8)
    yi = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(vi), 0.0884, causal=True, window=1))
    assert np.array_equal(yi, vi)


def test_sdp_attention_fused_kernel_structure(ops, oracle):
    import torch
    # first causal row attends to key 0 only: y[0] = v[0] exactly; a changed future key changes nothing before it
    heads, n, d = 2, 160, 128
    q, k, v = (synth.normal(s, (heads, n, d)).astype(np.float16) for s in (1, 2, 3))
    y = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0884, causal=True))
    assert np.array_equal(y[:, 0, :], v[:, 0, :])
    k2, v2 = k.copy(), v.copy()
    k2[:, 100:, :] += np.float16(1.0)
    v2[:, 100:, :] -= np.float16(2.0)
    y2 = host(ops.sdp_attention_fwd(dev(q), dev(k2), dev(v2), 0.0884, causal=True))
    assert np.array_equal(y[:, :100, :], y2[:, :100, :])
    assert not np.array_equal(y[:, 100:, :], y2[:, 100:, :])
    # constant v: every output equals that constant whatever the scores are
    vc = np.full_like(v, 0.5)
    yc = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(vc), 0.0884, softcap=20.0, causal=True, window=33))
    assert np.max(np.abs(yc.astype(np.float32) - 0.5)) <= 1e-3
    # more queries than keys with the causal rule: the first n_q - n_k queries see nothing and get zeros
    ys = host(ops.sdp_attention_fwd(dev(q), dev(k[:, :60]), dev(v[:, :60]), 0.0884, causal=True))
    assert not ys[:, :100, :].any() and ys[:, 100:, :].any()
    # against the three-launch form with the mask as data
    mask = oracle.slide_mask(oracle.causal_mask(n, n), 48).reshape(1, n, n)
    with np.errstate(over="ignore"):
        mask16 = mask.astype(np.float16)
    three = host(ops.sdp_attention_masked_scaled_fwd(dev(q), dev(k), dev(v), dev(mask16), 0.0884)).astype(np.float32)
    fused = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0884, causal=True, window=48)).astype(np.float32)
    assert scaled_rel_err(fused, three, 1.0) <= TOL_F16_ROWOPS * 2
    # rejected arguments launch nothing
    from anygpu_amd import capi
    lib = capi.load()
    t = torch.zeros((2, 16, 96), device="cuda", dtype=torch.float16)
    out = torch.full_like(t, 3.0)
    f = lib.anygpu_sdp_attention_fwd_f16
    assert f(t.data_ptr(), t.data_ptr(), t.data_ptr(), out.data_ptr(), 2, 1, 16, 16, 96, 0.1, 0.0, 1, 0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert f(t.data_ptr(), t.data_ptr(), t.data_ptr(), out.data_ptr(), 3, 2, 16, 16, 64, 0.1, 0.0, 1, 0, None) == capi.ANYGPU_ERR_BAD_SHAPE
    assert f(t.data_ptr(), None, t.data_ptr(), out.data_ptr(), 2, 1, 16, 16, 64, 0.1, 0.0, 1, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())


def test_sdp_attention_fused_kernel_many_heads_d128(ops, oracle):
    # enough query blocks at head_dim 128 for the 32-queries-per-wave form: 64 heads over 16 key / value heads,
    # 1000 queries at the end of 1100 keys, softcap + causal + window
    h, hkv, n_q, n_k, d = 64, 16, 1000, 1100, 128
    q = synth.normal(1, (h, n_q, d)).astype(np.float16)
    k = synth.normal(2, (hkv, n_k, d)).astype(np.float16)
    v = synth.normal(3, (hkv, n_k, d)).astype(np.float16)
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0884, softcap=30.0, causal=True, window=300)).astype(np.float32)
    idx = np.array([0, 1, 15, 16, 31, 32, 255, 256, 257, 511, 700, 998, 999], dtype=np.int64)
    want = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t) for t in (q, k, v)), alpha=0.0884, softcap=30.0,
                                      causal=True, window=300, q_per_kv=4, query_index=idx, threads=8)
    assert scaled_rel_err(got[:, idx, :], want, 1.0) <= TOL_F16_ROWOPS * 2
    # every query against the same kernel's 16-queries-per-wave form (fewer heads per launch take it)
    parts = [host(ops.sdp_attention_fwd(dev(q[i:i + 4]), dev(k[i // 4:i // 4 + 1]), dev(v[i // 4:i // 4 + 1]), 0.0884,
                                        softcap=30.0, causal=True, window=300)) for i in (0, 28, 60)]
    for i, part in zip((0, 28, 60), parts):
        assert scaled_rel_err(got[i:i + 4], part.astype(np.float32), 1.0) <= 2e-3


DECODE_CASES = [
    # heads, kv_heads, n_q, n_k, d, alpha, softcap, causal, window
    (8, 4, 1, 4500, 256, 0.0625, 50.0, True, 4096),       # Gemma2 generation step: window cuts the cache
    (32, 8, 1, 1000, 128, 0.0884, 0.0, True, 0),
    (16, 16, 1, 300, 64, 0.125, 0.0, False, 0),
    (8, 2, 4, 2049, 128, 0.0884, 0.0, True, 0),           # 4 query heads x 4 queries = 16 rows per key / value head
    (4, 4, 3, 777, 64, 0.125, 30.0, True, 100),
    (2, 1, 1, 63, 128, 0.0884, 0.0, True, 0),             # less than one tile of keys
    (4, 2, 5, 3, 64, 0.125, 0.0, True, 0),                # more queries than keys: the first two see nothing
    (4, 2, 1, 12000, 64, 0.125, 0.0, True, 0),            # 188 key tiles of 64: more splits than one wave of the merge holds
    # more than 16 rows per key / value head: groups of 16 rows, a wave each (the last group partly filled)
    (8, 1, 4, 3000, 64, 0.125, 0.0, True, 0),             # 32 rows: two groups
    (16, 2, 5, 2049, 128, 0.0884, 0.0, True, 0),          # 40 rows: 16 + 16 + 8
    (8, 1, 16, 1500, 256, 0.0625, 50.0, True, 700),       # 128 rows: eight groups, softcap and window
    (6, 2, 7, 900, 64, 0.125, 0.0, False, 0),             # 21 rows
]


@pytest.mark.parametrize("case", DECODE_CASES)
def test_sdp_attention_decode_form(ops, oracle, case):
    heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window = case
    q = synth.normal(1 + n_q, (1, heads, n_q, d)).astype(np.float16)
    k = synth.normal(2 + n_k, (1, kv_heads, n_k, d)).astype(np.float16)
    v = synth.normal(3 + d, (1, kv_heads, n_k, d)).astype(np.float16)
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window,
                                     decode=True)).astype(np.float32)
    want = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t)[0] for t in (q, k, v)), alpha=alpha, softcap=cap,
                                      causal=causal, window=window, q_per_kv=heads // kv_heads, threads=8)
    # a query that sees no key: the operator chain divides 0 by 0 (NaN), the kernels give zeros
    blind = np.isnan(want).all(axis=(0, 2))
    assert blind.sum() == (max(n_q - n_k, 0) if causal else 0)
    assert not got[0][:, blind, :].any()
    assert scaled_rel_err(got[0][:, ~blind, :], want[:, ~blind, :], 1.0) <= TOL_F16_ROWOPS * 2
    # and against the fused form of the same arguments
    fused = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window,
                                       decode=False)).astype(np.float32)
    assert scaled_rel_err(got, fused, 1.0) <= 2e-3


@pytest.mark.parametrize("case", DECODE_CASES)
def test_sdp_attention_decode_form_f32(ops, oracle, case):
    heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window = case
    q = synth.normal(1 + n_q, (1, heads, n_q, d))
    k = synth.normal(2 + n_k, (1, kv_heads, n_k, d))
    v = synth.normal(3 + d, (1, kv_heads, n_k, d))
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window, decode=True))
    want = oracle.sdp_attention_rules(q[0], k[0], v[0], alpha=alpha, softcap=cap, causal=causal, window=window,
                                      q_per_kv=heads // kv_heads, threads=8)
    blind = np.isnan(want).all(axis=(0, 2))
    assert blind.sum() == (max(n_q - n_k, 0) if causal else 0)
    assert got.dtype == np.float32 and not got[0][:, blind, :].any()
    assert scaled_rel_err(got[0][:, ~blind, :], want[:, ~blind, :], 1.0) <= TOL_F32
    fused = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=causal, window=window, decode=False))
    assert scaled_rel_err(got, fused, 1.0) <= TOL_F32


def test_sdp_attention_decode_f32_workspace_and_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    ws_bytes = lib.anygpu_sdp_attention_decode_f32_workspace_bytes
    # 4 key / value heads, 2 rows each, 4096 visible keys = 256 tiles of 16 -> 256 splits: 4 * 256 * 2 * (256 + 2) floats
    assert ws_bytes(8, 2, 1, 8192, 256, 1, 4096) == 4 * 256 * 2 * 258 * 4
    assert ws_bytes(8, 2, 1, 40, 256, 1, 0) == 4 * 3 * 2 * 258 * 4           # 3 tiles -> 3 splits
    assert ws_bytes(0, 1, 1, 100, 64, 1, 0) == 0
    assert ws_bytes(8, 2, 9, 100, 64, 1, 0) == 4 * 7 * 18 * 66 * 4           # 18 rows per key / value head: two groups; 7 tiles
    assert ws_bytes(8, 2, 65, 100, 64, 1, 0) == capi.ANYGPU_ERR_UNSUPPORTED  # 130 rows per key / value head
    q = torch.zeros((4, 1, 64), device="cuda")
    kv = torch.zeros((2, 500, 64), device="cuda")
    y = torch.full_like(q, 3.0)
    need = ws_bytes(4, 2, 1, 500, 64, 1, 0)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    f = lib.anygpu_sdp_attention_decode_f32
    args = (4, 2, 1, 500, 64, 0.125, 0.0, 1, 0, None)
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), None, need, *args) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), ws.data_ptr(), need - 1, *args) == capi.ANYGPU_ERR_BAD_SHAPE
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())


def test_sdp_attention_decode_workspace_and_rejected_arguments(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    ws_bytes = lib.anygpu_sdp_attention_decode_workspace_bytes
    # 4 key / value heads, 2 rows each, 4096 visible keys = 64 tiles -> 64 splits: 4 * 64 * 2 * (256 + 2) floats
    assert ws_bytes(8, 2, 1, 8192, 256, 1, 4096) == 4 * 64 * 2 * 258 * 4
    assert ws_bytes(8, 2, 1, 100, 256, 1, 0) == 4 * 2 * 2 * 258 * 4          # 2 tiles -> 2 splits
    assert ws_bytes(0, 1, 1, 100, 64, 1, 0) == 0
    assert ws_bytes(8, 2, 9, 100, 64, 1, 0) == 4 * 2 * 18 * 66 * 4           # 18 rows per key / value head: two groups; 2 tiles
    assert ws_bytes(8, 2, 65, 100, 64, 1, 0) == capi.ANYGPU_ERR_UNSUPPORTED  # 130 rows per key / value head
    assert ws_bytes(8, 3, 1, 100, 64, 1, 0) == capi.ANYGPU_ERR_BAD_SHAPE
    q = torch.zeros((4, 1, 64), device="cuda", dtype=torch.float16)
    kv = torch.zeros((2, 500, 64), device="cuda", dtype=torch.float16)
    y = torch.full_like(q, 3.0)
    need = ws_bytes(4, 2, 1, 500, 64, 1, 0)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    f = lib.anygpu_sdp_attention_decode_f16
    args = (4, 2, 1, 500, 64, 0.125, 0.0, 1, 0, None)
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), None, need, *args) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), ws.data_ptr(), need - 1, *args) == capi.ANYGPU_ERR_BAD_SHAPE
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), ws.data_ptr() + 4, need, *args) == capi.ANYGPU_ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())
    # a workspace larger than needed and reused by a second, smaller call
    big = torch.empty(need + 4096, dtype=torch.uint8, device="cuda")
    qr = torch.randn((4, 1, 64), device="cuda", dtype=torch.float16)
    kr = torch.randn((2, 500, 64), device="cuda", dtype=torch.float16)
    vr = torch.randn((2, 500, 64), device="cuda", dtype=torch.float16)
    for n_k in (500, 130):
        out = torch.empty_like(qr)
        kk, vv = kr[:, :n_k].contiguous(), vr[:, :n_k].contiguous()
        assert f(qr.data_ptr(), kk.data_ptr(), vv.data_ptr(), out.data_ptr(), big.data_ptr(), big.numel(),
                 4, 2, 1, n_k, 64, 0.125, 0.0, 1, 0, None) == capi.ANYGPU_OK
        ref = ops.sdp_attention_fwd(qr, kk, vv, 0.125, causal=True, decode=False)
        torch.cuda.synchronize()
        assert float((out.float() - ref.float()).abs().max()) <= 2e-3


def test_sdp_attention_fused_kernel_gemma2_block(ops, oracle):
    # Gemma2 attention at the softmax configuration of the headline set: 8 query heads over 4 key / value heads,
    # head_dim 256, scale 1 / 16, softcap 50, causal + window 4096; 6144 positions so that the window cuts
    h, hkv, n, d = 8, 4, 6144, 256
    q = synth.normal(1, (h, n, d)).astype(np.float16)
    k = synth.normal(2, (hkv, n, d)).astype(np.float16)
    v = synth.normal(3, (hkv, n, d)).astype(np.float16)
    got = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), 0.0625, softcap=50.0, causal=True, window=4096)).astype(np.float32)
    idx = np.array([0, 1, 63, 64, 127, 128, 1000, 4095, 4096, 4097, 5000, 6143], dtype=np.int64)
    want = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t) for t in (q, k, v)), alpha=0.0625, softcap=50.0,
                                      causal=True, window=4096, q_per_kv=2, query_index=idx, threads=8)
    assert scaled_rel_err(got[:, idx, :], want, 1.0) <= TOL_F16_ROWOPS * 2
    assert np.isfinite(got).all()


def test_sdp_attention_key_split_blocks_agree_with_whole_blocks(ops, oracle):
    # A windowed launch with at least a block per CU whose longest blocks are a large share of a CU's work is dispatched
    # with those blocks in two key halves plus a merge (partial results in the stream's K-split workspace).  With a
    # workspace too small for a single partial the same call runs whole blocks.  Both against the oracle, and against
    # each other to the rounding of the fp16 result; a ragged last query block and a head_dim of 128 included.
    import torch
    for h, hkv, n, d, win, cap in [(8, 4, 6144 - 40, 256, 2048, 50.0), (16, 8, 4096, 128, 1024, 0.0)]:
        q = synth.normal(1, (h, n, d)).astype(np.float16)
        k = synth.normal(2, (hkv, n, d)).astype(np.float16)
        v = synth.normal(3, (hkv, n, d)).astype(np.float16)
        alpha = 1.0 / math.sqrt(d)
        split = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=True, window=win)).astype(np.float32)
        tiny = torch.empty((64,), device="cuda")
        ops.set_workspace(tiny)
        try:
            whole = host(ops.sdp_attention_fwd(dev(q), dev(k), dev(v), alpha, softcap=cap, causal=True, window=win)).astype(np.float32)
        finally:
            torch.cuda.synchronize()
            ops.set_workspace(None)
        assert np.isfinite(split).all()
        assert scaled_rel_err(split, whole, 1.0) <= 2e-3
        assert not np.array_equal(split, whole), "the launch was expected to take the key-split path"
        idx = np.array([0, 127, 128, 1000, n - 2049, n - 2048, n - 1000, n - 129, n - 128, n - 1], dtype=np.int64)
        want = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t) for t in (q, k, v)), alpha=alpha, softcap=cap,
                                          causal=True, window=win, q_per_kv=h // hkv, query_index=idx, threads=8)
        assert scaled_rel_err(split[:, idx, :], want, 1.0) <= TOL_F16_ROWOPS * 2
        assert scaled_rel_err(whole[:, idx, :], want, 1.0) <= TOL_F16_ROWOPS * 2
        # the float32 kernel takes the same path
        q32, k32, v32 = (oracle.cvt_f16_to_f32(t) for t in (q, k, v))
        split32 = host(ops.sdp_attention_fwd(dev(q32), dev(k32), dev(v32), alpha, softcap=cap, causal=True, window=win))
        ops.set_workspace(tiny)
        try:
            whole32 = host(ops.sdp_attention_fwd(dev(q32), dev(k32), dev(v32), alpha, softcap=cap, causal=True, window=win))
        finally:
            torch.cuda.synchronize()
            ops.set_workspace(None)
        assert scaled_rel_err(split32, whole32, 1.0) <= TOL_F32
        assert scaled_rel_err(split32[:, idx, :], want, 1.0) <= TOL_F32


# =============================================================================================
# launches recorded into a HIP graph
# =============================================================================================

def _graph_problem(ops):
    import torch
    from anygpu_amd import capi
    a32 = torch.empty((24, 4096), device="cuda")
    w32 = dev(synth.uniform(1, (4096, 260)))                        # [K, N] fp32: band kernel, K split
    a16 = torch.empty((128, 2304), device="cuda", dtype=torch.float16)
    w16 = dev(synth.uniform(2, (2048, 2304)).astype(np.float16))    # [N, K] fp16: tile kernel, K split
    sc = torch.empty((64, 512), device="cuda", dtype=torch.float16)
    cx = torch.empty((2, 16, 300), device="cuda", dtype=torch.float16)
    cw, cb = dev(synth.normal(3, (16, 4)).astype(np.float16)), dev(synth.normal(4, (16,)).astype(np.float16))
    q = torch.empty((1, 4, 100, 128), device="cuda")
    kv = dev(synth.normal(5, (1, 2, 100, 128)))
    q16 = torch.empty((1, 4, 150, 256), device="cuda", dtype=torch.float16)     # head_dim 256: its own kernel
    kv16 = dev(synth.normal(6, (1, 2, 150, 256)).astype(np.float16))

    def fill(seed):
        a32.copy_(dev(synth.uniform(seed, tuple(a32.shape))))
        a16.copy_(dev(synth.uniform(seed + 1, tuple(a16.shape)).astype(np.float16)))
        sc.copy_(dev((synth.normal(seed + 2, tuple(sc.shape)) * np.float32(4.0)).astype(np.float16)))
        cx.copy_(dev(synth.normal(seed + 3, tuple(cx.shape)).astype(np.float16)))
        q.copy_(dev(synth.normal(seed + 4, tuple(q.shape))))
        q16.copy_(dev(synth.normal(seed + 5, tuple(q16.shape)).astype(np.float16)))

    def work():
        return (ops.tensor_mm(a32, w32),
                ops.tensor_mm(a16, w16, b_layout=capi.B_COL_MAJOR),
                ops.tensor_softmax(sc, alpha=0.125, causal=True, q_len=64),
                ops.tensor_causal_conv1d(cx, cw, cb),
                ops.sdp_attention_fwd(q, kv, kv, 0.0884, softcap=30.0, causal=True, window=40),
                ops.sdp_attention_fwd(q16, kv16, kv16, 0.0625, softcap=50.0, causal=True, window=70))

    return fill, work


def test_launches_replayed_from_a_graph_with_a_caller_workspace(ops, oracle):
    # A stream that has never run anything gets a caller's K-split workspace, the calls are captured on it and replayed
    # three times with new input values and eager work in between.  The library allocates nothing (free device memory
    # does not move), the workspace is written by the replays, and every replay equals the eager result of the default
    # stream bit for bit, because with a workspace of the same size both make the same cuts.
    import torch
    from anygpu_amd import capi
    fill, work = _graph_problem(ops)
    side = torch.cuda.Stream()
    ws_side = torch.full((capi.WORKSPACE_BYTES // 4,), float("nan"), device="cuda")
    ws_main = torch.empty((capi.WORKSPACE_BYTES // 4,), device="cuda")
    fill(10)
    torch.cuda.synchronize()
    ops.set_workspace(ws_side, side)
    ops.set_workspace(ws_main)
    try:
        work()                                                       # (torch's eager pool holds the result tensors from here on)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = work()
        for rep in range(3):
            fill(20 + 10 * rep)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = [host(t).copy() for t in outs]
            want = [host(t) for t in work()]                         # eager, on the default stream
            torch.cuda.synchronize()
            for g, w in zip(got, want):
                assert np.array_equal(g, w)
        assert not bool(torch.isnan(ws_side[:1024]).all()), "the replays did not use the workspace handed in"
        # (the graph's own pool holds the result tensors of work() and the runtime its graph: less than a 64 MiB workspace)
        assert free_before - torch.cuda.mem_get_info()[0] < capi.WORKSPACE_BYTES - (8 << 20)
    finally:
        torch.cuda.synchronize()
        ops.set_workspace(None, side)
        ops.set_workspace(None)


def test_key_split_attention_replayed_from_a_graph(ops):
    # The fused attention with its longest query blocks in two key halves (partial results in the caller's workspace, a
    # merge launch behind) recorded into a graph: every replay equals the eager result bit for bit, new queries each time.
    import torch
    from anygpu_amd import capi
    h, hkv, n, d, win, cap = 8, 4, 6144 - 40, 256, 2048, 50.0
    k = dev(synth.normal(2, (hkv, n, d)).astype(np.float16))
    v = dev(synth.normal(3, (hkv, n, d)).astype(np.float16))
    q = torch.empty((h, n, d), device="cuda", dtype=torch.float16)
    side = torch.cuda.Stream()
    ws_side = torch.full((capi.WORKSPACE_BYTES // 4,), float("nan"), device="cuda")
    ws_main = torch.empty((capi.WORKSPACE_BYTES // 4,), device="cuda")
    ops.set_workspace(ws_side, side)
    ops.set_workspace(ws_main)
    try:
        q.copy_(dev(synth.normal(10, (h, n, d)).astype(np.float16)))
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out = ops.sdp_attention_fwd(q, k, v, 0.0625, softcap=cap, causal=True, window=win)
        for rep in range(3):
            q.copy_(dev(synth.normal(20 + rep, (h, n, d)).astype(np.float16)))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = host(out).copy()
            want = host(ops.sdp_attention_fwd(q, k, v, 0.0625, softcap=cap, causal=True, window=win))
            torch.cuda.synchronize()
            assert np.isfinite(got.astype(np.float32)).all()
            assert np.array_equal(got, want)
        assert not bool(torch.isnan(ws_side[:1024]).all()), "the replays were expected to leave partial results in the workspace"
    finally:
        torch.cuda.synchronize()
        ops.set_workspace(None, side)
        ops.set_workspace(None)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_mask_tensor_attention_replayed_from_a_graph(ops, monkeypatch, dtype):
    # The attention with the mask as a tensor, with its pass over the mask (the note of hidden key tiles at the front of
    # the caller's workspace) and few query blocks in parts of their key range (partial results behind the note, a merge
    # launch), recorded into a graph: every replay equals the eager result bit for bit, with a new mask and new queries
    # each time and the library's eager work on another stream's workspace in between.  Without a workspace the captured
    # call takes neither the note nor the parts; the result agrees to rounding.
    import torch
    from anygpu_amd import capi
    tdt, ndt = (torch.float16, np.float16) if dtype == "f16" else (torch.float32, np.float32)
    h, n_q, n_k, d = 4, 200, 3000, 128
    k = dev(synth.normal(2, (1, h, n_k, d)).astype(ndt))
    v = dev(synth.normal(3, (1, h, n_k, d)).astype(ndt))
    q = torch.empty((1, h, n_q, d), device="cuda", dtype=tdt)
    mask = torch.empty((1, 1, n_q, n_k), device="cuda", dtype=tdt)

    def new_inputs(seed):
        rng = np.random.default_rng(seed)
        m = rng.normal(0.0, 1.0, (n_q, n_k)).astype(np.float32)
        hide_key_stripes(m, rng)
        with np.errstate(over="ignore"):
            mask.copy_(dev(m.astype(ndt)).reshape(1, 1, n_q, n_k))
        q.copy_(dev(synth.normal(seed, (1, h, n_q, d)).astype(ndt)))
        torch.cuda.synchronize()

    monkeypatch.setenv("ANYGPU_ATTN_MASK_MAP_FROM", "0")
    side = torch.cuda.Stream()
    ws_side = torch.full((capi.WORKSPACE_BYTES // 4,), float("nan"), device="cuda")
    ws_main = torch.empty((capi.WORKSPACE_BYTES // 4,), device="cuda")
    ops.set_workspace(ws_side, side)
    ops.set_workspace(ws_main)
    try:
        new_inputs(10)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out = ops.sdp_attention_masked_scaled_fwd(q, k, v, mask, d ** -0.5)
        ops.set_workspace(None, side)
        bare = torch.cuda.CUDAGraph()
        with torch.cuda.graph(bare, stream=side):
            out_bare = ops.sdp_attention_masked_scaled_fwd(q, k, v, mask, d ** -0.5)
        ops.set_workspace(ws_side, side)
        for rep in range(3):
            new_inputs(20 + rep)
            graph.replay()
            bare.replay()
            torch.cuda.synchronize()
            got, got_bare = host(out).copy(), host(out_bare).copy()
            want = host(ops.sdp_attention_masked_scaled_fwd(q, k, v, mask, d ** -0.5))
            torch.cuda.synchronize()
            assert np.isfinite(got.astype(np.float32)).all()
            assert np.array_equal(got, want)
            # (whole blocks instead of parts of the key range: another order of summation)
            assert np.allclose(got_bare.astype(np.float32), want.astype(np.float32), rtol=0.0, atol=2e-3 if dtype == "f16" else 2e-5)
        assert not bool(torch.isnan(ws_side[:64]).all()), "the replays were expected to leave the note of hidden tiles in the workspace"
    finally:
        torch.cuda.synchronize()
        ops.set_workspace(None, side)
        ops.set_workspace(None)


def test_captured_launches_without_a_workspace_run_uncut(ops, oracle):
    # Under capture the library's own workspace is never used, warmed up or not: every product runs uncut, which is what
    # an eager launch does whose workspace is too small for a single plane.  Both agree bit for bit, and with the cut
    # result of an ordinary eager launch to the rounding of another order of summation.
    import torch
    fill, work = _graph_problem(ops)
    side = torch.cuda.Stream()
    fill(10)
    with torch.cuda.stream(side):
        cut = [host(t).copy() for t in work()]                      # eager: allocates the stream's own workspace and cuts
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        outs = work()
    tiny = torch.empty((64,), device="cuda")
    ops.set_workspace(tiny)
    try:
        for rep in range(2):
            fill(10 if rep == 0 else 40)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = [host(t).copy() for t in outs]
            want = [host(t) for t in work()]                         # eager and uncut: the workspace holds no plane
            torch.cuda.synchronize()
            for g, w in zip(got, want):
                assert np.array_equal(g, w)
            if rep == 0:
                assert scaled_rel_err(got[0], cut[0], math.sqrt(4096) / 3.0) <= TOL_F32
                assert scaled_rel_err(got[1].astype(np.float32), cut[1].astype(np.float32), math.sqrt(2304) / 3.0) <= TOL_F16_GEMM
                assert not np.array_equal(got[0], cut[0]) or not np.array_equal(got[1], cut[1])
    finally:
        torch.cuda.synchronize()
        ops.set_workspace(None)
        ops.set_workspace(None, side)


def test_release_workspaces_returns_the_memory(ops):
    import torch
    from anygpu_amd import capi
    ops.release_workspaces()
    stream = torch.cuda.Stream()
    a = dev(synth.uniform(1, (24, 8192)))
    w = dev(synth.uniform(2, (260, 8192)))
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(stream):
        ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR)              # few rows, deep K: cut, into the library's own buffer
    torch.cuda.synchronize()
    free1 = torch.cuda.mem_get_info()[0]
    assert free0 - free1 >= capi.WORKSPACE_BYTES
    ops.release_workspaces()
    # (the runtime returns memory in granules of its own: a 2 MiB piece of the buffer may stay with a chunk it shares)
    assert torch.cuda.mem_get_info()[0] - free1 >= capi.WORKSPACE_BYTES * 7 // 8
    # and the stream simply gets a new one the next time
    with torch.cuda.stream(stream):
        again = ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR)
    assert np.isfinite(host(again)).all()
    ops.release_workspaces()


def test_library_owned_workspaces_are_bounded(ops):
    # streams come and go without the library seeing it: it keeps at most MAX_OWN_WORKSPACES buffers of its own, a
    # further stream takes the place of the one used longest ago
    import torch
    from anygpu_amd import capi
    ops.release_workspaces()
    a = dev(synth.uniform(1, (24, 8192)))
    w = dev(synth.uniform(2, (260, 8192)))
    want = host(ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR))
    ops.release_workspaces()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    streams = [torch.cuda.Stream() for _ in range(capi.MAX_OWN_WORKSPACES + 3)]
    outs = []
    for st in streams:
        with torch.cuda.stream(st):
            outs.append(ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR))     # few rows, deep K: cut, into the library's own buffer
    torch.cuda.synchronize()
    held = free0 - torch.cuda.mem_get_info()[0]
    assert held <= capi.MAX_OWN_WORKSPACES * capi.WORKSPACE_BYTES + (32 << 20), held
    assert held >= (capi.MAX_OWN_WORKSPACES - 1) * capi.WORKSPACE_BYTES
    for out in outs:
        assert np.array_equal(host(out), want)
    # the first streams lost their buffers to the later ones and simply get new ones
    with torch.cuda.stream(streams[0]):
        again = ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR)
    assert np.array_equal(host(again), want)
    ops.release_workspaces()


def test_mm_f32_operand_copies_larger_than_the_first_workspace(ops, oracle):
    # odd row pitches and a K that is no multiple of 32: both operands are copied, aligned and padded, into the stream's
    # workspace; the two copies (52 + 69 MB) exceed the 64 MiB the library allocates first, so its buffer grows.
    # Small integers: every sum is exact, whatever the order; torch.matmul on the same operands must agree bit for bit,
    # and a few rows are held against the oracle.
    import torch
    from anygpu_amd import capi
    ops.release_workspaces()
    m, k, n = 3000, 4099, 4095
    a = synth.integers(71, (m, k), -2, 2)
    w = synth.integers(72, (n, k), -2, 2)
    da, dw = dev(a), dev(w)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    got = ops.tensor_mm(da, dw, b_layout=capi.B_COL_MAJOR)
    torch.cuda.synchronize()
    held = free0 - torch.cuda.mem_get_info()[0] - got.numel() * 4
    assert capi.WORKSPACE_BYTES < held <= 3 * capi.WORKSPACE_BYTES, held       # 121 MB of copies in steps of 64 MiB
    assert torch.equal(got, torch.matmul(da, dw.t()))
    rows = [0, 1, 1499, 2999]
    want = mm_want(oracle, a[rows], np.ascontiguousarray(w.T))
    assert np.array_equal(host(got)[rows], want)
    # the grown buffer serves later calls, large and small
    free1 = torch.cuda.mem_get_info()[0]
    again = ops.tensor_mm(da, dw, b_layout=capi.B_COL_MAJOR)
    small = ops.tensor_mm(da[:24], dw[:260], b_layout=capi.B_COL_MAJOR)
    torch.cuda.synchronize()
    assert free1 - torch.cuda.mem_get_info()[0] <= again.numel() * 4 + (8 << 20)
    assert torch.equal(again, got) and torch.equal(small, got[:24, :260])
    ops.release_workspaces()


def test_k_split_products_on_concurrent_streams(ops, oracle):
    # every stream owns its partial-sum workspace: products that are cut along K may overlap on different streams
    import torch
    from anygpu_amd import capi
    streams = [torch.cuda.Stream() for _ in range(3)]
    problems = []
    for i, (m, k, n) in enumerate([(24, 8192, 260), (128, 4608, 512), (16, 9216, 2304)]):
        a = dev(synth.uniform(10 + i, (m, k)))
        w = dev(synth.uniform(20 + i, (n, k)))
        problems.append((a, w, host(ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR))))
    torch.cuda.synchronize()
    results = [[] for _ in streams]
    for rep in range(8):
        for si, st in enumerate(streams):
            a, w, _ = problems[(si + rep) % 3]
            with torch.cuda.stream(st):
                results[si].append(((si + rep) % 3, ops.tensor_mm(a, w, b_layout=capi.B_COL_MAJOR)))
    torch.cuda.synchronize()
    for per_stream in results:
        for which, out in per_stream:
            assert np.array_equal(host(out), problems[which][2])


# =============================================================================================
# committed golden fixtures (tests/golden/*.dat)
# =============================================================================================

def test_golden_fixtures_through_c_abi(ops):
    import sys
    from pathlib import Path
    golden = Path(__file__).resolve().parent / "golden"
    sys.path.insert(0, str(golden))
    from dat_codec import load_tensor

    d = golden / "test_causal_conv1d_fwd_f32"
    got = host(ops.tensor_causal_conv1d(dev(load_tensor(d / "x.dat")), dev(load_tensor(d / "w.dat")),
                                        dev(load_tensor(d / "b.dat"))))
    assert scaled_rel_err(got, load_tensor(d / "y.dat"), 1.0) <= TOL_F32

    d = golden / "test_mm_m24_n16_k40_f32"
    got = host(ops.tensor_mm(dev(load_tensor(d / "x.dat")), dev(load_tensor(d / "w.dat"))))
    assert scaled_rel_err(got, load_tensor(d / "y.dat"), math.sqrt(40) / 3.0) <= TOL_F32

    d = golden / "test_mm_m64_n64_k128_f16"
    got = host(ops.tensor_mm(dev(load_tensor(d / "x.dat")), dev(load_tensor(d / "w.dat")))).astype(np.float32)
    assert scaled_rel_err(got, load_tensor(d / "y.dat").astype(np.float32), math.sqrt(128) / 3.0) <= TOL_F16_GEMM

    d = golden / "test_softmax_masked_scaled_f32"
    want = load_tensor(d / "y.dat")
    got = host(ops.tensor_softmax(dev(load_tensor(d / "scores.dat")), alpha=0.125, causal=True, q_len=16))
    assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= TOL_F32
    assert np.all(got[np.tile(load_tensor(d / "mask.dat"), (2, 1)) != 0] == 0.0)

    d = golden / "test_softmax_softcap_window_f32"
    want = load_tensor(d / "y.dat")
    got = host(ops.tensor_softmax(dev(load_tensor(d / "scores.dat")), alpha=0.0625, softcap=50.0, causal=True,
                                  window=6, q_len=16))
    assert scaled_rel_err(got, want, want.max(axis=1, keepdims=True)) <= TOL_F32
    assert np.all(got[np.tile(load_tensor(d / "mask.dat"), (2, 1)) != 0] == 0.0)

    d = golden / "test_gemma2_lmhead_softcap"
    w = load_tensor(d / "gemma2_causal_lm.gemma2forcausallm.model.embed_tokens.weight.dat")
    got = host(ops.tensor_gemma_linear_softcap(dev(load_tensor(d / "in_0.dat")), dev(w), 30.0))
    assert scaled_rel_err(got, load_tensor(d / "out_0.dat"), 30.0) <= TOL_F32

    d = golden / "test_gemma2decoder_mlp"
    wg, wu, wd = (load_tensor(d / f"gemma2decoder_mlp.gemma2mlp.{n}_proj.weight.dat") for n in ("gate", "up", "down"))
    x = load_tensor(d / "in_0.dat")
    mid = ops.mlp_gemma2_fused_upproj(dev(x), dev(np.ascontiguousarray(wg.T)), dev(np.ascontiguousarray(wu.T)))
    from anygpu_amd import capi
    got = host(ops.tensor_mm(mid.reshape(-1, wd.shape[1]), dev(wd), b_layout=capi.B_COL_MAJOR)).reshape(x.shape)
    assert scaled_rel_err(got, load_tensor(d / "out_0.dat"), 1.0) <= TOL_F32

    d = golden / "test_mamba2layer_gated_rmsnorm"
    got = host(ops.tensor_zamba_gated_rmsnorm(dev(load_tensor(d / "in_0.dat")), dev(load_tensor(d / "in_1.dat")),
                                              dev(load_tensor(d / "mamba2layer_rmsnorm.rmsnorm.weight.dat")), 64, 1e-5))
    assert scaled_rel_err(got, load_tensor(d / "out_0.dat"), 1.0) <= TOL_F32

    d = golden / "test_causal_conv1d_update_f32"
    x, w, b = load_tensor(d / "x.dat"), load_tensor(d / "w.dat"), load_tensor(d / "b.dat")
    want = load_tensor(d / "y.dat")
    import torch
    state = torch.zeros((x.shape[0], x.shape[1], w.shape[1] - 1), device="cuda")
    for t in range(x.shape[2]):
        got = host(ops.tensor_causal_conv1d_update(dev(x[:, :, t]), state, dev(w), dev(b)))
        assert scaled_rel_err(got, want[:, :, t], 1.0) <= TOL_F32
    assert np.array_equal(host(state), load_tensor(d / "state.dat"))

    d = golden / "test_sdp_rules_f16_gqa"
    got = host(ops.sdp_attention_fwd(*(dev(load_tensor(d / f"{n}.dat")) for n in ("q", "k", "v")), 0.125, softcap=20.0,
                                     causal=True, window=12)).astype(np.float32)
    assert scaled_rel_err(got, load_tensor(d / "y.dat"), 1.0) <= TOL_F16_ROWOPS * 2

    d = golden / "test_sdp_rules_f32_d256"
    got = host(ops.sdp_attention_fwd(*(dev(load_tensor(d / f"{n}.dat")) for n in ("q", "k", "v")), 0.0625, softcap=50.0,
                                     causal=True, window=10))
    assert scaled_rel_err(got, load_tensor(d / "y.dat"), 1.0) <= TOL_F32
