#!/usr/bin/env python3
"""Writes the .dat fixtures under tests/golden/torch_* whose EXPECTED values come from PyTorch's
library routines evaluated in float64, not from the CPU oracle under oracle/.  Each case restates
the one-line torch formula the reference's own generator uses for that operator:

    scaled dot-product attention   F.scaled_dot_product_attention(q, k, v, mask, scale)   scripts/sdp_test_cases.py:162-171
    grouped-query form             the same on repeat_interleave'd k / v
    softcap + window softmax       softmax(where(visible, cap * tanh(alpha * x / cap), -inf)), window rule of
                                   scripts/gemma2/slide_mask_test.py:17-22 (tril(diagonal=-W) is masked)
    causal conv1d + SiLU           F.silu(F.conv1d(x, w.unsqueeze(1), b, padding=width-1, groups=dims))[..., :seq_len]
                                   scripts/fused_test_cases.py:41
    conv1d decode step             the same F.conv1d without padding over [state | new sample]: one output per row; the new
                                   state is the old one shifted by a sample (the step the Mamba2 mixer takes per token)
    gated RMS norm                 rms_norm(x * silu(z)) * w, srcs/models/zamba2/zamba_gated_rmsnorm.hpp:9-23
    matmul                         torch.matmul, scripts/mm_test_cases.py:18,42

Inputs are seeded synthetic tensors of a few KB (anygpu_amd.synth); nothing here imports oracle/.
Re-run from the repository root:   python tests/golden/make_torch_fixtures.py
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F

HERE = Path(__file__).resolve().parent
REPO = HERE.parent.parent
sys.path.insert(0, str(REPO))
sys.path.insert(0, str(HERE))

from anygpu_amd import synth  # noqa: E402
from dat_codec import save_tensor  # noqa: E402


def case_dir(name: str) -> Path:
    d = HERE / name
    d.mkdir(exist_ok=True)
    return d


def t64(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).double()


def f32(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.float32).numpy()


def visible(n_q: int, n_k: int, causal: bool, window: int) -> torch.Tensor:
    """Boolean [n_q, n_k]: query i (sitting at key position i + n_k - n_q) sees key j.  Causal: j <= position;
    window W: the keys tril(diagonal=-W) selects (j <= position - W) are masked as well."""
    shift = n_k - n_q
    ones = torch.ones(n_q, n_k, dtype=torch.bool)
    vis = ones.clone()
    if causal:
        vis &= ones.tril(diagonal=shift)
    if window > 0:
        vis &= ~ones.tril(diagonal=shift - window)
    return vis


def main() -> None:
    torch.manual_seed(0)

    # 1. the reference generator's case at a committed size: [1, heads, N, d], additive tril -inf mask, scale 0.125
    d = case_dir("torch_sdp_fwd_masked_scaled_f32")
    heads, n, dh = 4, 16, 128                                        # the generator's N = 16, d = 128 with 4 of its 32 heads
    q, k, v = (synth.normal(300 + i, (1, heads, n, dh)) for i in range(3))
    mask = torch.zeros(1, 1, n, n, dtype=torch.float64)
    mask.masked_fill_(torch.ones(1, 1, n, n, dtype=torch.bool).tril(diagonal=0).logical_not(), float("-inf"))
    y = F.scaled_dot_product_attention(t64(q), t64(k), t64(v), mask, scale=0.125)
    for name, t in (("q", q), ("k", k), ("v", v), ("mask", f32(mask))):
        save_tensor(t, d / f"{name}.dat")
    save_tensor(f32(y), d / "y.dat")

    # 2. grouped queries, more keys than queries, causal + window (no softcap: F.scaled_dot_product_attention itself):
    #    6 query heads over 2 key / value heads (3 per group), 20 queries at the end of 36 keys, d = 64, half inputs
    d = case_dir("torch_sdp_gqa_window_f16")
    hq, hkv, n_q, n_k, dh, win = 6, 2, 20, 36, 64, 9
    q = synth.normal(310, (1, hq, n_q, dh)).astype(np.float16)
    k = synth.normal(311, (1, hkv, n_k, dh)).astype(np.float16)
    v = synth.normal(312, (1, hkv, n_k, dh)).astype(np.float16)
    kk, vv = (t64(t.astype(np.float32)).repeat_interleave(hq // hkv, dim=1) for t in (k, v))
    y = F.scaled_dot_product_attention(t64(q.astype(np.float32)), kk, vv, visible(n_q, n_k, True, win), scale=0.125)
    for name, t in (("q", q), ("k", k), ("v", v)):
        save_tensor(t, d / f"{name}.dat")
    save_tensor(f32(y), d / "y.dat")

    # 3. grouped queries with the Gemma2 score transform: scale 1/16, softcap 50, causal + window, float32, d = 256,
    #    4 query heads over 2 key / value heads, 12 queries at the end of 40 keys
    d = case_dir("torch_sdp_gqa_softcap_window_f32_d256")
    hq, hkv, n_q, n_k, dh, win, cap, alpha = 4, 2, 12, 40, 256, 10, 50.0, 0.0625
    q = synth.normal(320, (1, hq, n_q, dh)) * np.float32(2.0)          # scores reach the cap's curved region
    k = synth.normal(321, (1, hkv, n_k, dh)) * np.float32(2.0)
    v = synth.normal(322, (1, hkv, n_k, dh))
    kk, vv = (t64(t).repeat_interleave(hq // hkv, dim=1) for t in (k, v))
    s = torch.matmul(t64(q), kk.transpose(-1, -2)) * alpha
    s = cap * torch.tanh(s / cap)
    s = torch.where(visible(n_q, n_k, True, win), s, torch.tensor(float("-inf"), dtype=torch.float64))
    y = torch.matmul(torch.softmax(s, dim=-1), vv)
    for name, t in (("q", q), ("k", k), ("v", v)):
        save_tensor(t, d / f"{name}.dat")
    save_tensor(f32(y), d / "y.dat")

    # 4. softmax of Gemma2 attention scores: [heads * q, k] rows, x 1/16, softcap 50, causal + window 6
    d = case_dir("torch_softmax_softcap_window_f32")
    heads, n_q, n_k, win, cap, alpha = 3, 16, 16, 6, 50.0, 0.0625
    x = synth.normal(330, (heads * n_q, n_k), std=16.0) * np.float32(4.0)
    z = cap * torch.tanh(t64(x) * alpha / cap)
    vis = visible(n_q, n_k, True, win).repeat(heads, 1)
    y = torch.softmax(torch.where(vis, z, torch.tensor(float("-inf"), dtype=torch.float64)), dim=-1)
    save_tensor(x, d / "scores.dat")
    save_tensor(f32(y), d / "y.dat")
    save_tensor(vis.to(torch.int32).numpy(), d / "visible.dat")

    # 4b. plain causal softmax of scaled scores (F.softmax of scale * x + additive -inf mask, scripts/sdp_test_cases.py:123)
    d = case_dir("torch_softmax_causal_scaled_f32")
    x = synth.normal(335, (2 * 24, 24), std=4.0)
    add = torch.zeros(24, 24, dtype=torch.float64).masked_fill_(~visible(24, 24, True, 0), float("-inf")).repeat(2, 1)
    save_tensor(x, d / "scores.dat")
    save_tensor(f32(F.softmax(t64(x) * 0.125 + add, dim=-1)), d / "y.dat")

    # 5. depthwise causal conv1d + SiLU, the generator's formula at a committed size (widths 4 and 3)
    for name, (b, dims, s, width), seed in (("torch_causal_conv1d_fwd_f32", (2, 7, 45, 4), 340),
                                            ("torch_causal_conv1d_fwd_w3_f32", (1, 5, 19, 3), 345)):
        d = case_dir(name)
        x, w, bias = synth.normal(seed, (b, dims, s)), synth.normal(seed + 1, (dims, width)), synth.normal(seed + 2, (dims,))
        y = F.silu(F.conv1d(t64(x), t64(w).unsqueeze(1), t64(bias), stride=1, padding=width - 1, groups=dims))[:, :, :s]
        save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat"); save_tensor(bias, d / "b.dat")
        save_tensor(f32(y), d / "y.dat")

    # 5b. the decode step: a state of width - 1 earlier samples (oldest first), one new sample per row
    for name, (b, dims, width), seed in (("torch_causal_conv1d_update_f32", (3, 11, 4), 347),
                                         ("torch_causal_conv1d_update_w2_f32", (2, 6, 2), 348)):
        d = case_dir(name)
        state, x = synth.normal(seed, (b, dims, width - 1)), synth.normal(seed + 10, (b, dims))
        w, bias = synth.normal(seed + 20, (dims, width)), synth.normal(seed + 30, (dims,))
        seq = torch.cat([t64(state), t64(x).unsqueeze(-1)], dim=-1)                       # [b, dims, width]
        y = F.silu(F.conv1d(seq, t64(w).unsqueeze(1), t64(bias), stride=1, padding=0, groups=dims))[:, :, 0]
        save_tensor(state, d / "state.dat"); save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat"); save_tensor(bias, d / "b.dat")
        save_tensor(f32(y), d / "y.dat"); save_tensor(f32(seq[:, :, 1:]), d / "new_state.dat")

    # 6. gated RMS norm of the Mamba2 mixer: rms_norm(x * silu(z), eps) * w over the last dimension
    d = case_dir("torch_gated_rmsnorm_f32")
    x = synth.normal(350, (1, 6, 96)); z = synth.normal(351, (1, 6, 96)) * np.float32(2.0)
    w = synth.uniform(352, (96,), 0.5, 1.5)
    g = t64(x) * F.silu(t64(z))
    y = F.rms_norm(g, (96,), t64(w), eps=1e-5)
    save_tensor(x, d / "in_0.dat"); save_tensor(z, d / "in_1.dat"); save_tensor(w, d / "weight.dat")
    save_tensor(f32(y), d / "out_0.dat")

    # 7. matmul, float32 and half inputs (torch.matmul in float64 on the stored values)
    d = case_dir("torch_mm_m24_n16_k40_f32")
    x, w = synth.uniform(360, (24, 40), 0.0, 1.0), synth.uniform(361, (40, 16), 0.0, 1.0)
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat"); save_tensor(f32(torch.matmul(t64(x), t64(w))), d / "y.dat")
    d = case_dir("torch_mm_m64_n64_k128_f16")
    x = synth.uniform(370, (64, 128)).astype(np.float16); w = synth.uniform(371, (128, 64)).astype(np.float16)
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat")
    save_tensor(f32(torch.matmul(t64(x.astype(np.float32)), t64(w.astype(np.float32)))), d / "y.dat")

    # 8. Gemma2 output head: softcap 30 on x @ W^T (torch.tanh), and the MLP's gelu_tanh(gate) * up
    d = case_dir("torch_gemma2_lmhead_softcap_f32")
    x = synth.normal(380, (5, 48)); w = synth.normal(381, (70, 48)) * np.float32(4.0)
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat")
    save_tensor(f32(30.0 * torch.tanh(F.linear(t64(x), t64(w)) / 30.0)), d / "y.dat")
    d = case_dir("torch_gemma2_mlp_upproj_f32")
    x = synth.normal(385, (7, 32)); wg = synth.normal(386, (96, 32)) * np.float32(0.3); wu = synth.normal(387, (96, 32)) * np.float32(0.3)
    save_tensor(x, d / "x.dat"); save_tensor(wg, d / "w_gate.dat"); save_tensor(wu, d / "w_up.dat")
    save_tensor(f32(F.gelu(F.linear(t64(x), t64(wg)), approximate="tanh") * F.linear(t64(x), t64(wu))), d / "y.dat")

    print("torch-sourced fixtures written under", HERE)


if __name__ == "__main__":
    main()
