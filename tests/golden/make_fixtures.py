#!/usr/bin/env python3
"""Writes the small .dat fixtures under tests/golden/ from seeded synthetic inputs and the CPU
oracle.  Folder and file names follow the reference's golden-test layout (one folder per case
with x.dat / w.dat / b.dat / y.dat ..., tests/ext_torch_tests.cpp:587-644,745-778), at sizes of
a few KB so that they can be committed.  Re-run from the repository root:
    python tests/golden/make_fixtures.py
The reference's own fixtures are not available (not in its repository, unseeded generator), so
expected outputs come from the oracle, which tests/test_oracle_pins.py ties down independently.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
REPO = HERE.parent.parent
sys.path.insert(0, str(REPO))
sys.path.insert(0, str(HERE))

import oracle  # noqa: E402
from anygpu_amd import synth  # noqa: E402
from dat_codec import save_tensor  # noqa: E402


def case_dir(name: str) -> Path:
    d = HERE / name
    d.mkdir(exist_ok=True)
    return d


def main() -> None:
    # causal conv1d + SiLU, float32: the reference case's layout at a committed size
    d = case_dir("test_causal_conv1d_fwd_f32")
    x = synth.normal(100, (2, 6, 40))
    w = synth.normal(101, (6, 4))
    b = synth.normal(102, (6,))
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat"); save_tensor(b, d / "b.dat")
    save_tensor(oracle.tensor_causal_conv1d(x, w, b), d / "y.dat")

    # float32 matmul (positive inputs like the reference's torch.rand case: elementwise rel 1 % gate)
    d = case_dir("test_mm_m24_n16_k40_f32")
    x = synth.uniform(110, (24, 40), 0.0, 1.0)
    w = synth.uniform(111, (40, 16), 0.0, 1.0)
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat")
    save_tensor(oracle.tensor_mm(x, w), d / "y.dat")

    # float16 matmul: half inputs, expected output = float32 oracle on the up-cast inputs, rounded to half
    d = case_dir("test_mm_m64_n64_k128_f16")
    x = synth.uniform(120, (64, 128), 0.0, 1.0).astype(np.float16)
    w = synth.uniform(121, (128, 64), 0.0, 1.0).astype(np.float16)
    y = oracle.tensor_mm(oracle.cvt_f16_to_f32(x), oracle.cvt_f16_to_f32(w))
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat"); save_tensor(y.astype(np.float16), d / "y.dat")

    # masked, scaled attention scores -> probabilities: [heads * q, k] scores, causal -inf mask, scale 0.125
    d = case_dir("test_softmax_masked_scaled_f32")
    heads, q, k = 2, 16, 16
    s = synth.normal(130, (heads * q, k), std=8.0)
    mask = oracle.causal_mask(q, k)
    save_tensor(s, d / "scores.dat"); save_tensor(mask, d / "mask.dat")
    save_tensor(oracle.attention_softmax(s, alpha=0.125, causal=True, q_len=q), d / "y.dat")

    # Gemma2-style: scale 1/16, softcap 50, causal + sliding window 6
    d = case_dir("test_softmax_softcap_window_f32")
    s = synth.normal(140, (heads * q, k), std=16.0)
    mask = oracle.slide_mask(oracle.causal_mask(q, k), 6)
    save_tensor(s, d / "scores.dat"); save_tensor(mask, d / "mask.dat")
    save_tensor(oracle.attention_softmax(s, alpha=0.0625, softcap=50.0, causal=True, window=6, q_len=q), d / "y.dat")

    # masked, scaled dot-product attention in the layout of the reference's golden case
    # (tests/ext_torch_tests.cpp:84-109: [1, heads, N, d], tril -inf mask, scale 0.125), small
    d = case_dir("test_sdp_fwd_masked_scaled_f32_16_32")
    heads, n, dh = 4, 16, 32
    q = synth.normal(150, (1, heads, n, dh)); k = synth.normal(151, (1, heads, n, dh)); v = synth.normal(152, (1, heads, n, dh))
    mask = oracle.causal_mask(n, n).reshape(1, 1, n, n)
    for name, t in (("q", q), ("k", k), ("v", v), ("mask", mask)):
        save_tensor(t, d / f"{name}.dat")
    save_tensor(oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask, 0.125), d / "y.dat")

    # Gemma2 output head with logit soft-capping, file names of tests/gemma2_tests.cpp:312-335
    d = case_dir("test_gemma2_lmhead_softcap")
    x = synth.normal(160, (1, 5, 48))
    w = synth.normal(161, (70, 48)) * np.float32(4.0)                     # [vocab, hidden]; logits reach past the cap of 30
    save_tensor(x, d / "in_0.dat"); save_tensor(w, d / "gemma2_causal_lm.gemma2forcausallm.model.embed_tokens.weight.dat")
    save_tensor(oracle.gemma_linear_softcap(x, w, 30.0), d / "out_0.dat")

    # Gemma2 MLP, gate / up / down weights stored [out, in] as in the reference's checkpoints (gemma_mlp.hpp:20-38
    # transposes them at load), tests/gemma2_tests.cpp:22-52
    d = case_dir("test_gemma2decoder_mlp")
    hidden, inter = 32, 96
    x = synth.normal(170, (1, 7, hidden))
    wg = synth.normal(171, (inter, hidden)) * np.float32(0.3)
    wu = synth.normal(172, (inter, hidden)) * np.float32(0.3)
    wd = synth.normal(173, (hidden, inter)) * np.float32(0.2)
    mid = oracle.gemma_mlp_upproj(x, np.ascontiguousarray(wg.T), np.ascontiguousarray(wu.T))
    y = oracle.tensor_mm(mid.reshape(7, inter), np.ascontiguousarray(wd.T)).reshape(1, 7, hidden)
    save_tensor(x, d / "in_0.dat")
    for name, t in (("gate_proj", wg), ("up_proj", wu), ("down_proj", wd)):
        save_tensor(t, d / f"gemma2decoder_mlp.gemma2mlp.{name}.weight.dat")
    save_tensor(y, d / "out_0.dat")

    # gated RMS norm of the Mamba2 mixer, tests/zamba2_tests.cpp:458-489 (eps 1e-5, one group = the row)
    d = case_dir("test_mamba2layer_gated_rmsnorm")
    x = synth.normal(180, (1, 6, 64)); z = synth.normal(181, (1, 6, 64)) * np.float32(2.0)
    w = synth.uniform(182, (64,), 0.5, 1.5)
    save_tensor(x, d / "in_0.dat"); save_tensor(z, d / "in_1.dat"); save_tensor(w, d / "mamba2layer_rmsnorm.rmsnorm.weight.dat")
    save_tensor(oracle.zamba_gated_rmsnorm(x, z, w, 1e-5), d / "out_0.dat")

    # decode steps of the causal convolution: the columns of x one at a time, state carried along
    d = case_dir("test_causal_conv1d_update_f32")
    x = synth.normal(190, (2, 6, 9)); w = synth.normal(191, (6, 4)); b = synth.normal(192, (6,))
    save_tensor(x, d / "x.dat"); save_tensor(w, d / "w.dat"); save_tensor(b, d / "b.dat")
    save_tensor(oracle.tensor_causal_conv1d(x, w, b), d / "y.dat")     # column t is the output of step t
    save_tensor(np.ascontiguousarray(x[:, :, -3:]), d / "state.dat")   # the state after the last step

    # attention with rule masks, half precision inputs: 4 query heads over 2 key / value heads, 24 queries at the end
    # of 40 keys, d = 64, scale 0.125, softcap 20, causal + window 12
    d = case_dir("test_sdp_rules_f16_gqa")
    q = synth.normal(200, (1, 4, 24, 64)).astype(np.float16)
    k = synth.normal(201, (1, 2, 40, 64)).astype(np.float16)
    v = synth.normal(202, (1, 2, 40, 64)).astype(np.float16)
    y = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t)[0] for t in (q, k, v)), alpha=0.125, softcap=20.0,
                                   causal=True, window=12, q_per_kv=2)
    for name, t in (("q", q), ("k", k), ("v", v)):
        save_tensor(t, d / f"{name}.dat")
    save_tensor(y.reshape(1, 4, 24, 64), d / "y.dat")

    # the same rules in float32 at head dimension 256 (the reference's fused kernel is float32, d = 256): 2 query heads
    # over 1 key / value head, 20 queries at the end of 36 keys, scale 1/16, softcap 50, causal + window 10
    d = case_dir("test_sdp_rules_f32_d256")
    q = synth.normal(210, (1, 2, 20, 256))
    k = synth.normal(211, (1, 1, 36, 256))
    v = synth.normal(212, (1, 1, 36, 256))
    y = oracle.sdp_attention_rules(q[0], k[0], v[0], alpha=0.0625, softcap=50.0, causal=True, window=10, q_per_kv=2)
    for name, t in (("q", q), ("k", k), ("v", v)):
        save_tensor(t, d / f"{name}.dat")
    save_tensor(y.reshape(1, 2, 20, 256), d / "y.dat")

    print("fixtures written under", HERE)


if __name__ == "__main__":
    main()
