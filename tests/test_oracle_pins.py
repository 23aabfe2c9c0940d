"""Pins the CPU oracle against what the mathematics fixes: closed forms, invariants, special
cases and independent brute force.  The reference holds no golden vectors for this path (its
.dat fixtures are not in the repository and came from an unseeded generator), so these checks
are what ties the oracle down; each is chosen so that a plausible slip (dropped term, wrong
sign or index, transposed operand, wrong tap order) fails at least one of them.
"""
import math

import numpy as np
import pytest

from anygpu_amd import synth


# ---------------------------------------------------------------------------------------------
# tensor_mm / tensor_gemm
# ---------------------------------------------------------------------------------------------

def test_mm_integer_inputs_bit_exact_vs_int64(oracle):
    # values 0..10 and K <= 2304 keep every partial sum below 2^24: float32 sums are exact,
    # so any correct implementation agrees bit for bit with integer arithmetic
    for (m, k, n, sa, sb) in [(40, 30, 50, 11, 18), (64, 2304, 33, 1, 2), (7, 1, 5, 3, 4)]:
        a = synth.integers(sa, (m, k), 0, 10)
        b = synth.integers(sb, (k, n), 0, 10)
        want = a.astype(np.int64) @ b.astype(np.int64)
        got = oracle.tensor_mm(a, b)
        assert np.array_equal(got.astype(np.int64), want)
        gi = oracle.tensor_mm(a.astype(np.int32), b.astype(np.int32))
        assert np.array_equal(gi.astype(np.int64), want)


def test_mm_non_square_catches_transposed_operands(oracle):
    # a product of distinct primes per position: swapping or transposing an operand changes the result
    a = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)            # 2 x 3
    b = np.array([[7, 8, 9, 10], [11, 12, 13, 14], [15, 16, 17, 18]], dtype=np.float32)  # 3 x 4
    want = np.array([[74, 80, 86, 92], [173, 188, 203, 218]], dtype=np.float32)
    assert np.array_equal(oracle.tensor_mm(a, b), want)


def test_mm_identity_ones_pattern(oracle):
    n = 37
    eye = np.eye(n, dtype=np.float32)
    x = synth.normal(5, (n, n))
    assert np.array_equal(oracle.tensor_mm(eye, x), x)
    assert np.array_equal(oracle.tensor_mm(x, eye), x)
    ones = np.ones((9, 123), dtype=np.float32)
    assert np.array_equal(oracle.tensor_mm(ones, ones.T.copy()), np.full((9, 9), 123, dtype=np.float32))
    # crt_pattern_tensor: element ix holds ix % 10 (srcs/core/tensor.hpp:514-528)
    pa = (np.arange(6 * 20) % 10).astype(np.float32).reshape(6, 20)
    pb = (np.arange(20 * 4) % 10).astype(np.float32).reshape(20, 4)
    want = np.array([[sum(((r * 20 + l) % 10) * ((l * 4 + c) % 10) for l in range(20)) for c in range(4)]
                     for r in range(6)], dtype=np.float32)
    assert np.array_equal(oracle.tensor_mm(pa, pb), want)


def test_mm_strided_views_equal_explicit_copies(oracle):
    a = synth.normal(1, (17, 29))
    bt = synth.normal(2, (23, 29))          # B stored [N, K]
    via_view = oracle.tensor_mm(a, bt.T)    # strides (1, K): column-major B
    via_copy = oracle.tensor_mm(a, np.ascontiguousarray(bt.T))
    assert np.array_equal(via_view, via_copy)
    wide = synth.normal(3, (17, 64))
    assert np.array_equal(oracle.tensor_mm(wide[:, :29], bt.T), oracle.tensor_mm(wide[:, :29].copy(), bt.T))


def test_mm_normal_inputs_within_float32_summation_bound(oracle):
    m, k, n = 33, 512, 41
    a = synth.normal(0, (m, k))
    b = synth.normal(1, (k, n))
    got = oracle.tensor_mm(a, b).astype(np.float64)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    bound = k * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64))
    assert np.all(np.abs(got - exact) <= bound)
    # and it is the sequential float32 sum, not a pairwise or float64 one
    seq = np.zeros((m, n), dtype=np.float32)
    for l in range(k):
        seq += np.outer(a[:, l], b[l, :]).astype(np.float32)
    assert np.array_equal(oracle.tensor_mm(a, b), seq)


def test_mm_float64_elements_use_float32_accumulator(oracle):
    a = synth.normal(3, (5, 300)).astype(np.float64)
    b = synth.normal(4, (300, 6)).astype(np.float64)
    got = oracle.tensor_mm(a, b)
    acc = np.zeros((5, 6), dtype=np.float32)
    for l in range(300):
        acc = (acc.astype(np.float64) + np.outer(a[:, l], b[l, :])).astype(np.float32)
    assert np.array_equal(got, acc.astype(np.float64))


def test_mm_row_range_and_threads_do_not_change_values(oracle):
    a = synth.normal(6, (64, 100))
    b = synth.normal(7, (100, 48))
    full = oracle.tensor_mm(a, b)
    part = oracle.tensor_mm(a, b, rows=(10, 20))
    assert np.array_equal(part[10:20], full[10:20]) and not part[:10].any() and not part[20:].any()
    assert np.array_equal(oracle.tensor_mm(a, b, threads=4), full)


def test_gemm_bias_is_added_per_column(oracle):
    x = synth.integers(1, (6, 9), 0, 10)
    w = synth.integers(2, (9, 4), 0, 10)
    b = np.array([1, 20, 300, 4000], dtype=np.float32)
    want = (x.astype(np.int64) @ w.astype(np.int64) + b.astype(np.int64)[None, :]).astype(np.float32)
    assert np.array_equal(oracle.tensor_gemm(x, w, b), want)


# ---------------------------------------------------------------------------------------------
# tensor_softmax and the prologue primitives
# ---------------------------------------------------------------------------------------------

def test_softmax_rows_sum_to_one_and_shift_invariant(oracle):
    x = synth.normal(0, (13, 257), std=3.0)
    y = oracle.tensor_softmax(x)
    assert np.all(np.abs(y.sum(axis=1, dtype=np.float64) - 1.0) <= 257 * 2.0 ** -24)
    assert np.all(y >= 0)
    x8 = np.round(x * 8) / 8          # multiples of 1/8: adding 4 is exact in float32
    assert np.array_equal(oracle.tensor_softmax(x8), oracle.tensor_softmax(x8 + np.float32(4.0)))


def test_softmax_constant_rows_are_exactly_one_over_n(oracle):
    for n in (1, 2, 64, 1024):
        x = np.full((3, n), 1.75, dtype=np.float32)
        assert np.array_equal(oracle.tensor_softmax(x), np.full((3, n), 1.0 / n, dtype=np.float32))


def test_softmax_two_values_closed_form_and_order(oracle):
    for delta in (0.5, 1.0, 3.25, 10.0):
        x = np.array([[0.0, delta], [delta, 0.0]], dtype=np.float32)
        y = oracle.tensor_softmax(x).astype(np.float64)
        big = 1.0 / (1.0 + math.exp(-delta))
        assert abs(y[0, 1] - big) < 2e-7 and abs(y[0, 0] - (1 - big)) < 2e-7
        assert abs(y[1, 0] - big) < 2e-7 and abs(y[1, 1] - (1 - big)) < 2e-7


def test_softmax_one_hot_limit_and_masked_entries_are_exact_zero(oracle):
    x = np.array([[0.0, 200.0, -5.0], [-np.inf, 2.0, -np.inf], [np.finfo(np.float32).min, 1.0, 1.0]], dtype=np.float32)
    y = oracle.tensor_softmax(x)
    assert np.array_equal(y[0], np.array([0, 1, 0], dtype=np.float32))
    assert np.array_equal(y[1], np.array([0, 1, 0], dtype=np.float32))
    assert np.array_equal(y[2], np.array([0, 0.5, 0.5], dtype=np.float32))


def test_softmax_vs_long_double_brute_force(oracle):
    x = synth.normal(4, (9, 61), std=2.0)
    y = oracle.tensor_softmax(x)
    xl = x.astype(np.longdouble)
    e = np.exp(xl - xl.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(y.astype(np.longdouble) - want)) < 61 * 2.0 ** -23
    y64 = oracle.tensor_softmax(x.astype(np.float64))
    assert np.max(np.abs(y64.astype(np.longdouble) - want)) < 1e-15


def test_softmax_strided_input(oracle):
    big = synth.normal(5, (6, 40))
    assert np.array_equal(oracle.tensor_softmax(big[:, :31]), oracle.tensor_softmax(big[:, :31].copy()))
    # column step: softmax over every second element
    assert np.array_equal(oracle.tensor_softmax(big[:, ::2]), oracle.tensor_softmax(big[:, ::2].copy()))


def test_mul_and_add_are_elementwise(oracle):
    x = synth.normal(1, (4, 5))
    y = synth.normal(2, (4, 5))
    assert np.array_equal(oracle.tensor_mul_scalar(x, 0.125), x * np.float32(0.125))
    assert np.array_equal(oracle.tensor_add(x, y), x + y)


def test_softcap_properties(oracle):
    cap = 50.0
    x = synth.normal(3, (1000,), std=40.0)
    y = oracle.softcap(x, cap)
    assert np.array_equal(oracle.softcap(-x, cap), -y)                        # odd
    assert np.all(np.abs(y) <= cap) and np.all(np.abs(y[np.abs(x) < 100]) < cap)
    assert np.all(np.sign(y) == np.sign(x))
    want = cap * np.tanh(x.astype(np.float64) / cap)
    assert np.max(np.abs(y - want)) < 1e-5 * cap
    half = np.array([cap * math.atanh(0.5)], dtype=np.float32)
    assert abs(float(oracle.softcap(half, cap)[0]) - cap / 2) < 1e-5 * cap
    tiny = np.array([1e-3, -2e-3], dtype=np.float32)
    assert np.allclose(oracle.softcap(tiny, cap), tiny, rtol=1e-6)              # y -> x as x/cap -> 0
    # a different cap changes the value: cap is not ignored, and it is not tanh(x) * cap
    assert abs(float(oracle.softcap(np.array([30.0], dtype=np.float32), 30.0)[0]) - 30 * math.tanh(1.0)) < 1e-4


def test_causal_and_slide_mask_rules(oracle):
    q = k = 9
    cm = oracle.causal_mask(q, k)
    for i in range(q):
        for j in range(k):
            assert cm[i, j] == (0.0 if j <= i else -np.inf)
    # sliding window: row i keeps keys {j : i - W < j <= i}; count = min(i + 1, W)
    window = 4
    sm = oracle.slide_mask(cm[None, None], window)[0, 0]
    lowest = np.finfo(np.float32).min
    for i in range(q):
        visible = [j for j in range(k) if sm[i, j] == 0.0]
        assert visible == [j for j in range(k) if i - window < j <= i]
        assert len(visible) == min(i + 1, window)
        for j in range(k):
            if j <= i - window:
                assert sm[i, j] == lowest
    # the generator's shape: [5, 1, 121, 41] with W = 34; rule == tril(diagonal=-W)
    rng_mask = synth.normal(8, (5, 1, 121, 41))
    out = oracle.slide_mask(rng_mask, 34)
    tril = np.tril(np.ones((121, 41), dtype=bool), k=-34)
    want = np.where(tril[None, None], lowest, rng_mask)
    assert np.array_equal(out, want)


def test_attention_softmax_is_the_stated_composition(oracle):
    rows, cols, q_len = 24, 12, 12
    x = synth.normal(2, (rows, cols), std=16.0)
    alpha, cap, window = 1.0 / 16.0, 50.0, 5
    got = oracle.attention_softmax(x, alpha=alpha, softcap=cap, causal=True, window=window, q_len=q_len)
    # composed by hand from the separately pinned primitives
    s = oracle.tensor_mul_scalar(x, alpha)
    s = oracle.softcap(s, cap).reshape(rows, cols)
    mask = oracle.slide_mask(oracle.causal_mask(q_len, cols), window)
    mask = np.tile(mask, (rows // q_len, 1))
    want = oracle.tensor_softmax(oracle.tensor_add(s, mask))
    assert np.array_equal(got, want)
    # float64 brute force of the same formula
    z = cap * np.tanh(x.astype(np.float64) * alpha / cap)
    i = (np.arange(rows) % q_len)[:, None]
    j = np.arange(cols)[None, :]
    vis = (j <= i) & (j > i - window)
    z = np.where(vis, z, -np.inf)
    e = np.exp(z - z.max(axis=1, keepdims=True))
    brute = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(got - brute)) < 1e-6
    assert np.all(got[~vis] == 0.0)
    assert got[0, 0] == 1.0 and not got[0, 1:].any()       # first causal row is [1, 0, ...]
    # row subset returns exactly those rows
    idx = np.array([3, 17, 23])
    sub = oracle.attention_softmax(x, alpha=alpha, softcap=cap, causal=True, window=window, q_len=q_len, row_index=idx)
    assert np.array_equal(sub, got[idx])
    # without softcap / masks it is plain softmax of the scaled input
    plain = oracle.attention_softmax(x, alpha=0.125)
    assert np.array_equal(plain, oracle.tensor_softmax(oracle.tensor_mul_scalar(x, 0.125)))


def test_sdp_attention_masked_scaled_vs_float64_formula(oracle):
    # the reference generator's case: [1, 32, N, d] with a tril -inf mask and scale 0.125
    # (scripts/sdp_test_cases.py:150-171, N = 16, d = 128 in tests/ext_torch_tests.cpp:86)
    heads, n, d = 32, 16, 128
    q = synth.normal(1, (1, heads, n, d))
    k = synth.normal(2, (1, heads, n, d))
    v = synth.normal(3, (1, heads, n, d))
    mask = oracle.causal_mask(n, n).reshape(1, 1, n, n)
    y = oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask, 0.125, threads=4)
    q64, k64, v64 = (t.astype(np.float64) for t in (q, k, v))
    s = 0.125 * np.einsum("bhqd,bhkd->bhqk", q64, k64) + mask.astype(np.float64)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    want = np.einsum("bhqk,bhkd->bhqd", e / e.sum(axis=-1, keepdims=True), v64)
    assert np.max(np.abs(y - want)) < 2e-5
    assert np.array_equal(y[:, :, 0, :], v[:, :, 0, :])       # the first causal row attends to key 0 only
    # the chain of primitives, one head
    h = 5
    qk = oracle.tensor_mm(q[0, h], k[0, h].T)
    chain = oracle.tensor_mm(oracle.tensor_softmax(oracle.tensor_add(oracle.tensor_mul_scalar(qk, 0.125), mask[0, 0])),
                             v[0, h])
    assert np.array_equal(y[0, h], chain)
    # rectangular: more keys than queries, window-style finite mask values
    q2, k2, v2 = synth.normal(4, (3, 5, 8)), synth.normal(5, (3, 9, 8)), synth.normal(6, (3, 9, 8))
    m2 = oracle.slide_mask(oracle.causal_mask(5, 9, diag=4), 3)
    y2 = oracle.sdp_attention_masked_scaled_fwd(q2, k2, v2, m2, 0.3)
    s2 = 0.3 * np.einsum("hqd,hkd->hqk", q2.astype(np.float64), k2.astype(np.float64))
    s2 = np.where(m2[None] == 0, s2, -np.inf)
    e2 = np.exp(s2 - s2.max(axis=-1, keepdims=True))
    want2 = np.einsum("hqk,hkd->hqd", e2 / e2.sum(axis=-1, keepdims=True), v2.astype(np.float64))
    assert np.max(np.abs(y2 - want2)) < 1e-5


def _attention_rules_float64(q, k, v, alpha, softcap, causal, window, q_per_kv):
    """Independent float64 evaluation, one (head, query) at a time with explicit loops over the visible key set."""
    heads, n_q, d = q.shape
    n_k = k.shape[1]
    out = np.zeros((heads, n_q, d))
    for h in range(heads):
        g = h // q_per_kv                                   # consecutive query heads share a key / value head
        for i in range(n_q):
            pos = i + (n_k - n_q)                           # the query's own key position
            keys = [j for j in range(n_k)
                    if (not causal or j <= pos) and (window <= 0 or j > pos - window)]
            if not keys:
                continue
            s = np.array([alpha * float(np.dot(q[h, i].astype(np.float64), k[g, j].astype(np.float64))) for j in keys])
            if softcap > 0:
                s = softcap * np.tanh(s / softcap)
            e = np.exp(s - s.max())
            p = e / e.sum()
            out[h, i] = sum(p[t] * v[g, j].astype(np.float64) for t, j in enumerate(keys))
    return out


@pytest.mark.parametrize("q_per_kv", [1, 2, 3])
def test_sdp_attention_rules_vs_float64_brute_force(oracle, q_per_kv):
    # more keys than queries (the diagonal sits at n_k - n_q), softcap, causal + window, grouped queries
    kv_heads, n_q, n_k, d = 2, 7, 19, 16
    heads = kv_heads * q_per_kv
    q = synth.normal(40, (heads, n_q, d)) * np.float32(1.5)
    k = synth.normal(41, (kv_heads, n_k, d)) * np.float32(1.5)
    v = synth.normal(42, (kv_heads, n_k, d))
    for kw in (dict(alpha=0.25, softcap=5.0, causal=True, window=6),
               dict(alpha=0.25, softcap=0.0, causal=True, window=0),
               dict(alpha=0.5, softcap=0.0, causal=False, window=0),
               dict(alpha=0.25, softcap=3.0, causal=True, window=25)):
        got = oracle.sdp_attention_rules(q, k, v, q_per_kv=q_per_kv, **kw)
        want = _attention_rules_float64(q, k, v, q_per_kv=q_per_kv, **kw)
        assert np.max(np.abs(got - want)) < 2e-6, kw
    # the value heads really differ, so a wrong head mapping cannot pass: h % kv_heads instead of h // q_per_kv
    if q_per_kv > 1:
        kw = dict(alpha=0.25, softcap=5.0, causal=True, window=6)
        got = oracle.sdp_attention_rules(q, k, v, q_per_kv=q_per_kv, **kw)
        wrong = np.stack([_attention_rules_float64(q[h:h + 1], k[h % kv_heads:h % kv_heads + 1],
                                                   v[h % kv_heads:h % kv_heads + 1], q_per_kv=1, **kw)[0]
                          for h in range(heads)])
        assert np.max(np.abs(got - wrong)) > 1e-2
    # a diagonal at 0 instead of n_k - n_q (the queries taken for the FIRST positions) gives different rows
    kw = dict(alpha=0.25, softcap=0.0, causal=True, window=0)
    got = oracle.sdp_attention_rules(q, k, v, q_per_kv=q_per_kv, **kw)
    first = _attention_rules_float64(q, k[:, :n_q], v[:, :n_q], q_per_kv=q_per_kv, **kw)
    assert np.max(np.abs(got - first)) > 1e-2
    # the last query sees every key when only the causal rule applies: plain softmax attention over all keys
    full = _attention_rules_float64(q[:, -1:], k, v, alpha=0.25, softcap=0.0, causal=False, window=0, q_per_kv=q_per_kv)
    assert np.max(np.abs(got[:, -1:] - full)) < 2e-6
    # a subset of queries returns exactly those rows
    idx = np.array([0, 3, 6])
    sub = oracle.sdp_attention_rules(q, k, v, q_per_kv=q_per_kv, query_index=idx, **kw)
    assert np.array_equal(sub, got[:, idx])


def test_sdp_attention_rules_equal_the_mask_tensor_form(oracle):
    # with one query head per key / value head the rule masks are the additive masks of the reference's chain:
    # square scores with the slide mask (its rule carries no diagonal shift, gemma_slide_mask.cu:21) ...
    heads, n, d = 3, 14, 8
    q, k, v = synth.normal(43, (heads, n, d)), synth.normal(44, (heads, n, d)), synth.normal(45, (heads, n, d))
    mask = oracle.slide_mask(oracle.causal_mask(n, n), 5)
    a = oracle.sdp_attention_rules(q, k, v, alpha=0.3, causal=True, window=5)
    assert np.array_equal(a, oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask, 0.3))
    # ... and more keys than queries with the causal mask shifted to the last queries
    n_q = 9
    mask = oracle.causal_mask(n_q, n, diag=n - n_q)
    a = oracle.sdp_attention_rules(q[:, :n_q], k, v, alpha=0.3, causal=True)
    assert np.array_equal(a, oracle.sdp_attention_masked_scaled_fwd(q[:, :n_q], k, v, mask, 0.3))


# ---------------------------------------------------------------------------------------------
# tensor_causal_conv1d
# ---------------------------------------------------------------------------------------------

def _silu64(v):
    v = np.asarray(v, dtype=np.float64)
    return v / (1.0 + np.exp(-v))


def test_conv1d_impulse_response_reads_taps_backwards(oracle):
    b, d, s, w = 1, 3, 10, 4
    x = np.zeros((b, d, s), dtype=np.float32)
    x[:, :, 0] = 1.0
    wt = np.array([[1, 2, 3, 4], [-1, 0.5, 0.25, 2], [0.1, 0.2, 0.3, 0.4]], dtype=np.float32)
    bt = np.array([0.5, -0.25, 0.0], dtype=np.float32)
    y = oracle.tensor_causal_conv1d(x, wt, bt)
    for ch in range(d):
        for t in range(s):
            pre = (wt[ch, w - 1 - t] if t < w else 0.0) + bt[ch]
            assert abs(y[0, ch, t] - _silu64(pre)) < 1e-6


def test_conv1d_special_weights(oracle):
    b, d, s = 2, 5, 33
    x = synth.normal(1, (b, d, s))
    bt = synth.normal(2, (d,), std=0.1)
    w_pass = np.zeros((d, 4), dtype=np.float32)
    w_pass[:, 3] = 1.0                                  # only the current-sample tap
    y = oracle.tensor_causal_conv1d(x, w_pass, bt)
    assert np.max(np.abs(y - _silu64(x.astype(np.float64) + bt[None, :, None]))) < 1e-6
    w_zero = np.zeros((d, 4), dtype=np.float32)
    y0 = oracle.tensor_causal_conv1d(x, w_zero, bt)
    assert np.max(np.abs(y0 - _silu64(bt)[None, :, None])) < 1e-6
    w_delay = np.zeros((d, 4), dtype=np.float32)
    w_delay[:, 0] = 1.0                                 # tap 0 is the sample three steps back
    yd = oracle.tensor_causal_conv1d(x, w_delay, np.zeros(d, dtype=np.float32))
    assert np.max(np.abs(yd[:, :, 3:] - _silu64(x[:, :, :-3]))) < 1e-6
    assert not yd[:, :, :3].any()                       # silu(0) = 0 in the padded region


def test_conv1d_is_causal_and_depthwise(oracle):
    b, d, s = 2, 4, 40
    x = synth.normal(3, (b, d, s))
    wt = synth.normal(4, (d, 4), std=0.5)
    bt = synth.normal(5, (d,), std=0.1)
    y = oracle.tensor_causal_conv1d(x, wt, bt)
    x2 = x.copy()
    x2[1, 2, 17] += 1.0
    y2 = oracle.tensor_causal_conv1d(x2, wt, bt)
    changed = np.argwhere(y != y2)
    assert set(map(tuple, changed)) == {(1, 2, 17), (1, 2, 18), (1, 2, 19), (1, 2, 20)}


def test_conv1d_vs_float64_zero_padded_brute_force(oracle):
    for width in (1, 2, 3, 4):
        b, d, s = 2, 7, 29
        x = synth.normal(6, (b, d, s))
        wt = synth.normal(7, (d, width), std=0.5)
        bt = synth.normal(8, (d,), std=0.1)
        y = oracle.tensor_causal_conv1d(x, wt, bt)
        xp = np.concatenate([np.zeros((b, d, width - 1)), x.astype(np.float64)], axis=2)
        pre = np.zeros((b, d, s))
        for k in range(width):
            pre += wt[None, :, k, None].astype(np.float64) * xp[:, :, k:k + s]
        pre += bt[None, :, None]
        assert np.max(np.abs(y - _silu64(pre))) < 2e-6
        y64 = oracle.tensor_causal_conv1d(x.astype(np.float64), wt.astype(np.float64), bt.astype(np.float64))
        assert np.max(np.abs(y64 - _silu64(pre))) < 1e-14


def test_conv1d_preactivation_is_linear_in_x(oracle):
    # with zero bias and small inputs silu is invertible on the image; compare pre-activations
    b, d, s = 1, 3, 20
    x1 = synth.integers(1, (b, d, s), -3, 3)
    x2 = synth.integers(2, (b, d, s), -3, 3)
    wt = synth.integers(3, (d, 4), -2, 2)
    zero = np.zeros(d, dtype=np.float32)

    def pre(x):
        # integer taps and samples: recover the exact integer pre-activation by brute force
        xp = np.concatenate([np.zeros((b, d, 3)), x], axis=2)
        return sum(wt[None, :, k, None] * xp[:, :, k:k + s] for k in range(4))

    for x in (x1, x2, x1 + x2):
        y = oracle.tensor_causal_conv1d(x.astype(np.float32), wt, zero)
        assert np.max(np.abs(y - _silu64(pre(x)))) < 1e-5
    assert np.array_equal(pre(x1 + x2), pre(x1) + pre(x2))


def test_conv1d_reference_generator_shape_vs_torch_formula(oracle):
    # scripts/fused_test_cases.py:31-41: batch 8, dims 2318, seq_len 638, width 4 and the one-line torch formula
    torch = pytest.importorskip("torch")
    import torch.nn.functional as F
    b, d, s, width = 8, 2318, 638, 4
    x = synth.normal(10, (b, d, s))
    wt = synth.normal(11, (d, width))
    bt = synth.normal(12, (d,))
    y = oracle.tensor_causal_conv1d(x, wt, bt, threads=8)
    tx, tw, tb = (torch.from_numpy(v).double() for v in (x, wt, bt))
    want = F.silu(F.conv1d(tx, tw.unsqueeze(1), tb, stride=1, padding=width - 1, groups=d))[:, :, :s].numpy()
    assert np.max(np.abs(y - want)) < 1e-5
    ok, _ = oracle.compare_data_buffers(y, want.astype(np.float32))      # the reference's own gate: abs 1e-3
    assert ok


# ---------------------------------------------------------------------------------------------
# GEMM epilogues: Gemma2 output head with logit soft-capping, MLP gate / up projections
# ---------------------------------------------------------------------------------------------

def test_linear_softcap_one_hot_rows_select_weight_entries(oracle):
    # x = e_h0 for every row: acc is a single product 1 * w[v, h0], so y[s, v] = softcap(w[v, h0]) exactly
    n, hsize, vsize, cap = 3, 11, 7, 30.0
    w = synth.normal(1, (vsize, hsize)) * np.float32(40.0)
    for h0 in (0, 5, 10):
        x = np.zeros((1, n, hsize), dtype=np.float32)
        x[..., h0] = 1.0
        y = oracle.gemma_linear_softcap(x, w, cap)
        assert y.shape == (1, n, vsize)
        want = oracle.softcap(w[:, h0], cap)
        assert np.array_equal(y, np.broadcast_to(want, (1, n, vsize)))
    # a transposed weight index (w[h, v]) or a row/column swap of y would fail the shapes above (7 != 11)


def test_linear_softcap_vs_float64_and_vs_mm_chain(oracle):
    n, hsize, vsize, cap = 9, 130, 37, 30.0
    x = synth.normal(2, (2, n, hsize))
    w = synth.normal(3, (vsize, hsize)) * np.float32(3.0)
    y = oracle.gemma_linear_softcap(x, w, cap, threads=4)
    logits = x.astype(np.float64).reshape(-1, hsize) @ w.astype(np.float64).T
    want = cap * np.tanh(logits / cap)
    assert np.abs(logits).max() > cap                      # the cap bites somewhere
    assert np.max(np.abs(y.reshape(-1, vsize) - want)) < 2e-5 * cap
    assert np.all(np.abs(y) < cap)
    # same sums as tensor_mm over the [hsize, vsize] strided view of w, then the scalar softcap
    chain = oracle.softcap(oracle.tensor_mm(x.reshape(-1, hsize), w.T), cap)
    assert np.array_equal(y.reshape(-1, vsize), chain)


def test_gelu_tanh_closed_forms(oracle):
    x = np.array([0.0, 1.0, -1.0, 10.0, -10.0, 0.5, -3.0], dtype=np.float32)
    y = oracle.tensor_gelu_tanh(x)
    assert y[0] == 0.0
    assert y[3] == 10.0 and abs(y[4]) == 0.0                # tanh saturates to +-1 in float32
    # gelu(x) - gelu(-x) = x / 2 * (tanh(u) - tanh(-u)) + x = x for the tanh form: tanh is odd
    grid = np.linspace(-6, 6, 4001).astype(np.float32)
    g = oracle.tensor_gelu_tanh(grid).astype(np.float64)
    gm = oracle.tensor_gelu_tanh(-grid).astype(np.float64)
    assert np.max(np.abs(g - gm - grid)) < 1e-6
    g64 = grid.astype(np.float64)
    want = 0.5 * g64 * (1 + np.tanh(math.sqrt(2 / math.pi) * (g64 + 0.044715 * g64 ** 3)))
    assert np.max(np.abs(g - want)) < 1e-6
    from scipy.special import erf
    exact = 0.5 * g64 * (1 + erf(g64 / math.sqrt(2)))
    assert np.max(np.abs(g - exact)) < 1e-3
    assert abs(y[1] - 0.841192) < 1e-5                      # published value of the tanh form at 1


def test_mlp_upproj_equals_primitive_chain_and_float64(oracle):
    n, hsize, isize = 7, 96, 50
    x = synth.normal(4, (1, n, hsize))
    wg = synth.normal(5, (hsize, isize)) * np.float32(0.2)
    wu = synth.normal(6, (hsize, isize)) * np.float32(0.2)
    y = oracle.gemma_mlp_upproj(x, wg, wu, threads=4)
    assert y.shape == (1, n, isize)
    x2 = x.reshape(n, hsize)
    chain = oracle.tensor_mul(oracle.tensor_gelu_tanh(oracle.tensor_mm(x2, wg)), oracle.tensor_mm(x2, wu))
    assert np.array_equal(y.reshape(n, isize), chain)
    g = x2.astype(np.float64) @ wg.astype(np.float64)
    u = x2.astype(np.float64) @ wu.astype(np.float64)
    want = 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3))) * u
    assert np.max(np.abs(y.reshape(n, isize) - want)) < 1e-4 * max(1.0, np.abs(want).max())
    # gate and up are not interchangeable: swapping them changes the result
    assert not np.allclose(oracle.gemma_mlp_upproj(x, wu, wg), y, atol=1e-3)


# ---------------------------------------------------------------------------------------------
# Mamba2 neighbours of the convolution: gated RMS norm, decode step of the convolution
# ---------------------------------------------------------------------------------------------

def test_silu_closed_forms(oracle):
    grid = np.linspace(-20, 20, 4001).astype(np.float32)
    s = oracle.tensor_silu(grid).astype(np.float64)
    sm = oracle.tensor_silu(-grid).astype(np.float64)
    assert oracle.tensor_silu(np.zeros(1, dtype=np.float32))[0] == 0.0
    assert np.max(np.abs(s - sm - grid)) < 2e-6                     # x s(x) - (-x) s(-x) = x (s(x) + s(-x)) = x
    g64 = grid.astype(np.float64)
    assert np.max(np.abs(s - g64 / (1 + np.exp(-g64)))) < 2e-6


def test_rms_norm_closed_forms(oracle):
    n = 64
    w = synth.uniform(1, (n,), 0.5, 1.5)
    # constant rows: mean x^2 = c^2 exactly, y = w c / sqrt(c^2 + eps)
    for c, eps in ((2.0, 1e-5), (-0.5, 0.0), (3.0, 1.0)):
        y = oracle.tensor_rms_norm(np.full((3, n), c, dtype=np.float32), w, eps)
        want = w.astype(np.float64) * c / math.sqrt(c * c + eps)
        assert np.max(np.abs(y - want)) < 1e-6
    x = synth.normal(2, (5, n))
    y0 = oracle.tensor_rms_norm(x, w, 0.0)
    assert np.max(np.abs(((y0 / w).astype(np.float64) ** 2).sum(axis=1) - n)) < 1e-3      # unit mean square
    assert np.max(np.abs(oracle.tensor_rms_norm(x * np.float32(4.0), w, 0.0) - y0)) < 1e-5  # scale invariance (x4 is exact)
    assert np.array_equal(oracle.tensor_rms_norm(x, w, 1e-5, zero_centered=True),
                          oracle.tensor_rms_norm(x, w + np.float32(1.0), 1e-5))
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * w
    assert np.max(np.abs(oracle.tensor_rms_norm(x, w, 1e-5) - want)) < 1e-5
    # a norm taken over the wrong axis or with the weight indexed by row would fail the shapes: w spans the last axis
    with pytest.raises(AssertionError):
        oracle.tensor_rms_norm(x.T.copy(), w, 1e-5)


def test_gated_rmsnorm_equals_chain_and_float64(oracle):
    rows, n, eps = 6, 96, 1e-5
    x, z = synth.normal(1, (rows, n)), synth.normal(2, (rows, n)) * np.float32(2.0)
    w = synth.uniform(3, (n,), 0.5, 1.5)
    y = oracle.zamba_gated_rmsnorm(x, z, w, eps)
    chain = oracle.tensor_rms_norm(oracle.tensor_mul(x, oracle.tensor_silu(z)), w, eps)
    assert np.array_equal(y, chain)
    x64, z64 = x.astype(np.float64), z.astype(np.float64)
    g = x64 * z64 / (1 + np.exp(-z64))
    want = g / np.sqrt((g ** 2).mean(axis=1, keepdims=True) + eps) * w
    assert np.max(np.abs(y - want)) < 1e-5
    assert not np.any(oracle.zamba_gated_rmsnorm(x, np.zeros_like(z), w, eps))            # silu(0) = 0 closes the gate
    # the gate is on z, not on x: swapping the two changes the result
    assert not np.allclose(oracle.zamba_gated_rmsnorm(z, x, w, eps), y, atol=1e-3)


def test_conv1d_update_steps_reproduce_whole_sequence(oracle):
    for width in (1, 2, 3, 4):
        b, d, s = 2, 5, 19
        x = synth.normal(width, (b, d, s))
        wt = synth.normal(10 + width, (d, width))
        bt = synth.normal(20 + width, (d,))
        full = oracle.tensor_causal_conv1d(x, wt, bt)
        state = np.zeros((b, d, width - 1), dtype=np.float32)
        for t in range(s):
            y, state = oracle.causal_conv1d_update(x[:, :, t], state, wt, bt)
            assert np.array_equal(y, full[:, :, t]), (width, t)
        assert np.array_equal(state, x[:, :, s - (width - 1):] if width > 1 else state)


# ---------------------------------------------------------------------------------------------
# fp16 up-cast and comparators
# ---------------------------------------------------------------------------------------------

def test_f16_upcast_all_bit_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.cvt_f16_to_f32(bits.view(np.float16))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)) or \
        np.array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_comparators_hand_computed(oracle):
    e = np.array([1.0, 2.0, 4.0], dtype=np.float32)
    a = np.array([1.0005, 2.0, 3.9995], dtype=np.float32)
    ok, worst = oracle.compare_data_buffers(a, e)                 # abs tol 1e-3
    assert ok and abs(worst - 5e-4) < 1e-6
    ok, _ = oracle.compare_data_buffers(a, e, abs_tol=4e-4)
    assert not ok
    a2 = np.array([1.02, 2.0, 4.0], dtype=np.float32)
    ok, worst = oracle.compare_data_buffers_reldiff(a2, e)        # 2 % off on the first element
    assert not ok and abs(worst - 0.02) < 1e-5
    ok, worst = oracle.compare_data_buffers_reldiff(np.array([1.005, 2.0, 4.0], dtype=np.float32), e)
    assert ok and abs(worst - 0.005) < 1e-5
    ok, val = oracle.compare_data_buffers_l2(a2, e)               # sqrt(0.0004 / 21)
    assert ok and abs(val - math.sqrt(0.0004 / 21.0)) < 1e-6
    ok, val = oracle.compare_data_buffers_l2(np.array([2.0, 2.0, 4.0], dtype=np.float32), e)
    assert not ok and abs(val - math.sqrt(1.0 / 21.0)) < 1e-6
