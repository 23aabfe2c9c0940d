"""The committed .dat fixtures are what tests/golden/make_fixtures.py produces (so the generator
and the data cannot drift apart) and the oracle reproduces every expected output."""
import sys
from pathlib import Path

import numpy as np

GOLDEN = Path(__file__).resolve().parent / "golden"
sys.path.insert(0, str(GOLDEN))

from dat_codec import load_tensor, save_tensor  # noqa: E402


def test_codec_roundtrip_and_byte_layout(tmp_path):
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    save_tensor(x, tmp_path / "t.dat")
    raw = (tmp_path / "t.dat").read_bytes()
    assert np.frombuffer(raw[:20], dtype="<i4").tolist() == [3, 2, 3, 4, 5]      # dim, shape, code FLOAT32
    assert len(raw) == 20 + 24 * 4
    assert np.array_equal(load_tensor(tmp_path / "t.dat"), x)
    h = x.astype(np.float16)
    save_tensor(h, tmp_path / "h.dat")
    assert np.frombuffer((tmp_path / "h.dat").read_bytes()[16:20], dtype="<i4")[0] == 4
    assert np.array_equal(load_tensor(tmp_path / "h.dat"), h)


def test_fixtures_match_the_oracle(oracle):
    d = GOLDEN / "test_causal_conv1d_fwd_f32"
    y = oracle.tensor_causal_conv1d(load_tensor(d / "x.dat"), load_tensor(d / "w.dat"), load_tensor(d / "b.dat"))
    assert np.array_equal(y, load_tensor(d / "y.dat"))
    d = GOLDEN / "test_mm_m24_n16_k40_f32"
    assert np.array_equal(oracle.tensor_mm(load_tensor(d / "x.dat"), load_tensor(d / "w.dat")), load_tensor(d / "y.dat"))
    d = GOLDEN / "test_mm_m64_n64_k128_f16"
    y = oracle.tensor_mm(oracle.cvt_f16_to_f32(load_tensor(d / "x.dat")), oracle.cvt_f16_to_f32(load_tensor(d / "w.dat")))
    assert np.array_equal(y.astype(np.float16), load_tensor(d / "y.dat"))
    d = GOLDEN / "test_sdp_fwd_masked_scaled_f32_16_32"
    q, k, v, mask = (load_tensor(d / f"{n}.dat") for n in ("q", "k", "v", "mask"))
    assert np.array_equal(oracle.sdp_attention_masked_scaled_fwd(q, k, v, mask, 0.125), load_tensor(d / "y.dat"))
    d = GOLDEN / "test_gemma2_lmhead_softcap"
    w = load_tensor(d / "gemma2_causal_lm.gemma2forcausallm.model.embed_tokens.weight.dat")
    assert np.array_equal(oracle.gemma_linear_softcap(load_tensor(d / "in_0.dat"), w, 30.0), load_tensor(d / "out_0.dat"))
    d = GOLDEN / "test_gemma2decoder_mlp"
    wg, wu, wd = (load_tensor(d / f"gemma2decoder_mlp.gemma2mlp.{n}_proj.weight.dat") for n in ("gate", "up", "down"))
    x = load_tensor(d / "in_0.dat")
    mid = oracle.gemma_mlp_upproj(x, np.ascontiguousarray(wg.T), np.ascontiguousarray(wu.T))
    y = oracle.tensor_mm(mid.reshape(-1, wd.shape[1]), np.ascontiguousarray(wd.T)).reshape(x.shape)
    assert np.array_equal(y, load_tensor(d / "out_0.dat"))
    # torch's library formula for the block: down(gelu_tanh(gate(x)) * up(x)) with [out, in] weights
    import torch
    import torch.nn.functional as F
    tx, tg, tu, td = (torch.from_numpy(t).double() for t in (x, wg, wu, wd))
    ref = F.linear(F.gelu(F.linear(tx, tg), approximate="tanh") * F.linear(tx, tu), td).numpy()
    assert np.max(np.abs(y - ref)) < 1e-5
    d = GOLDEN / "test_mamba2layer_gated_rmsnorm"
    x, z, w = load_tensor(d / "in_0.dat"), load_tensor(d / "in_1.dat"), load_tensor(d / "mamba2layer_rmsnorm.rmsnorm.weight.dat")
    y = oracle.zamba_gated_rmsnorm(x, z, w, 1e-5)
    assert np.array_equal(y, load_tensor(d / "out_0.dat"))
    g = torch.from_numpy(x).double() * F.silu(torch.from_numpy(z).double())
    ref = (g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + 1e-5) * torch.from_numpy(w).double()).numpy()
    assert np.max(np.abs(y - ref)) < 1e-5
    d = GOLDEN / "test_causal_conv1d_update_f32"
    x, w, b = load_tensor(d / "x.dat"), load_tensor(d / "w.dat"), load_tensor(d / "b.dat")
    state = np.zeros((x.shape[0], x.shape[1], w.shape[1] - 1), dtype=np.float32)
    want = load_tensor(d / "y.dat")
    for t in range(x.shape[2]):
        yt, state = oracle.causal_conv1d_update(x[:, :, t], state, w, b)
        assert np.array_equal(yt, want[:, :, t])
    assert np.array_equal(state, load_tensor(d / "state.dat"))
    d = GOLDEN / "test_sdp_rules_f16_gqa"
    q, k, v = (oracle.cvt_f16_to_f32(load_tensor(d / f"{n}.dat"))[0] for n in ("q", "k", "v"))
    y = oracle.sdp_attention_rules(q, k, v, alpha=0.125, softcap=20.0, causal=True, window=12, q_per_kv=2)
    assert np.array_equal(y.reshape(1, 4, 24, 64), load_tensor(d / "y.dat"))
    d = GOLDEN / "test_sdp_rules_f32_d256"
    q, k, v = (load_tensor(d / f"{n}.dat")[0] for n in ("q", "k", "v"))
    y = oracle.sdp_attention_rules(q, k, v, alpha=0.0625, softcap=50.0, causal=True, window=10, q_per_kv=2)
    assert np.array_equal(y.reshape(1, 2, 20, 256), load_tensor(d / "y.dat"))
    for name, kw in [("test_softmax_masked_scaled_f32", dict(alpha=0.125, causal=True, q_len=16)),
                     ("test_softmax_softcap_window_f32", dict(alpha=0.0625, softcap=50.0, causal=True, window=6, q_len=16))]:
        d = GOLDEN / name
        y = oracle.attention_softmax(load_tensor(d / "scores.dat"), **kw)
        assert np.array_equal(y, load_tensor(d / "y.dat"))
        # the stored additive mask is the one the kernel parameters describe
        mask = load_tensor(d / "mask.dat")
        assert np.all(y[np.tile(mask, (2, 1)) != 0] == 0)
        # torch's library formula on the same data: softmax(scale * s [capped] + mask)
        import torch
        s = torch.from_numpy(load_tensor(d / "scores.dat")).double() * kw["alpha"]
        if kw.get("softcap"):
            s = kw["softcap"] * torch.tanh(s / kw["softcap"])
        ref = torch.softmax(s + torch.from_numpy(np.tile(mask, (2, 1))).double(), dim=-1).numpy()
        assert np.max(np.abs(y - ref)) < 1e-6
