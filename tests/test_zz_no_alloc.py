"""The entry point that allocates nothing: anygpu_sdp_attention_decode_f16_static keeps the partial results of the
decode attention in a fixed device array of the library instead of a caller workspace.  Same kernels and split plan
as anygpu_sdp_attention_decode_f16, so the results have to be bit-identical, also on a second, smaller call that
finds the first call's contents in the array.  The file's name makes it the last one pytest collects.
"""
import numpy as np
import pytest

from anygpu_amd import synth

pytestmark = pytest.mark.gpu

GRANULE = 2 << 20      # the runtime hands device memory out and takes it back in pieces of 2 MiB


def _operands(heads, kv_heads, n_q, n_k, d, seed):
    import torch
    q = torch.from_numpy(synth.normal(seed, (heads, n_q, d)).astype(np.float16)).cuda()
    k = torch.from_numpy(synth.normal(seed + 1, (kv_heads, n_k, d)).astype(np.float16)).cuda()
    v = torch.from_numpy(synth.normal(seed + 2, (kv_heads, n_k, d)).astype(np.float16)).cuda()
    return q, k, v


def test_decode_static_scratch_matches_workspace_form_on_two_calls(ops, oracle):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    # the set-up call: an empty problem looks up the array's address on this device and launches nothing
    assert lib.anygpu_sdp_attention_decode_f16_static(None, None, None, None, 0, 1, 1, 100, 64, 0.125, 0.0, 1, 0, None) == capi.ANYGPU_OK
    cases = [
        # heads, kv_heads, n_q, n_k, d, alpha, softcap, causal, window: the Gemma2 generation step, then a smaller call
        (8, 4, 1, 6000, 256, 0.0625, 50.0, 1, 4096),
        (4, 2, 3, 777, 64, 0.125, 0.0, 1, 0),
    ]
    for i, (heads, kv_heads, n_q, n_k, d, alpha, cap, causal, window) in enumerate(cases):
        q, k, v = _operands(heads, kv_heads, n_q, n_k, d, 40 + 10 * i)
        shape = (heads, heads // kv_heads, n_q, n_k, d)
        need = lib.anygpu_sdp_attention_decode_workspace_bytes(*shape, causal, window)
        assert 0 < need <= capi.DECODE_STATIC_SCRATCH_BYTES
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = torch.full_like(q, 7.0)
        got = torch.full_like(q, 9.0)
        assert lib.anygpu_sdp_attention_decode_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), want.data_ptr(), ws.data_ptr(), need,
                                                   *shape, alpha, cap, causal, window, None) == capi.ANYGPU_OK
        torch.cuda.synchronize()
        # free device memory as the driver reports it: sees an allocation by the library or the runtime (queue scratch
        # of a kernel with a private segment), which torch's own allocator statistics would not
        free_before = torch.cuda.mem_get_info()[0]
        allocated_before = torch.cuda.memory_allocated()
        assert lib.anygpu_sdp_attention_decode_f16_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(),
                                                          *shape, alpha, cap, causal, window, None) == capi.ANYGPU_OK
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == allocated_before
        assert free_before - torch.cuda.mem_get_info()[0] < GRANULE, "device memory was allocated during the call"
        assert torch.equal(got, want), f"case {i}: static-scratch form differs from the workspace form"
        # and the workspace form itself against the oracle (fp16 row-op tolerance, doubled for the two roundings of p)
        ref = oracle.sdp_attention_rules(*(oracle.cvt_f16_to_f32(t.cpu().numpy()) for t in (q, k, v)), alpha=alpha, softcap=cap,
                                         causal=bool(causal), window=window, q_per_kv=heads // kv_heads, threads=8)
        assert float(np.abs(got.float().cpu().numpy() - ref).max()) <= 4e-3


def test_decode_static_scratch_rejects_what_does_not_fit(ops):
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    # 64 key / value heads x 16 splits x 16 rows x (256 + 2) floats = 16.9 MB: more than the array holds
    shape = (64, 1, 16, 4096, 256)
    assert lib.anygpu_sdp_attention_decode_workspace_bytes(*shape, 1, 0) > capi.DECODE_STATIC_SCRATCH_BYTES
    q = torch.zeros((64, 16, 256), device="cuda", dtype=torch.float16)
    kv = torch.zeros((64, 4096, 256), device="cuda", dtype=torch.float16)
    y = torch.full_like(q, 3.0)
    f = lib.anygpu_sdp_attention_decode_f16_static
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), *shape, 0.0625, 0.0, 1, 0, None) == capi.ANYGPU_ERR_SCRATCH_TOO_SMALL
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), None, 4, 2, 1, 500, 256, 0.0625, 0.0, 1, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert f(q.data_ptr(), kv.data_ptr(), kv.data_ptr(), y.data_ptr(), 8, 2, 65, 100, 64, 0.125, 0.0, 1, 0, None) == capi.ANYGPU_ERR_UNSUPPORTED   # 130 rows
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())


def test_decode_static_scratch_replayed_from_a_graph(ops):
    # the use the entry point is for: captured into a graph (no allocation may happen under capture), replayed several
    # times with eager work and synchronisations in between, every replay equal to the eager result bit for bit
    import torch
    from anygpu_amd import capi
    lib = capi.load()
    f = lib.anygpu_sdp_attention_decode_f16_static
    assert f(None, None, None, None, 0, 1, 1, 100, 64, 0.125, 0.0, 1, 0, None) == capi.ANYGPU_OK      # set-up call, outside capture
    heads, kv_heads, n_q, n_k, d = 8, 4, 1, 5000, 256
    q, k, v = _operands(heads, kv_heads, n_q, n_k, d, 70)
    shape = (heads, heads // kv_heads, n_q, n_k, d)
    eager = torch.full_like(q, 5.0)
    assert f(q.data_ptr(), k.data_ptr(), v.data_ptr(), eager.data_ptr(), *shape, 0.0625, 50.0, 1, 4096, None) == capi.ANYGPU_OK
    torch.cuda.synchronize()
    out = torch.full_like(q, 6.0)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.graph(graph, stream=side):
        rc = f(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), *shape, 0.0625, 50.0, 1, 4096,
               torch.cuda.current_stream().cuda_stream)
    assert rc == capi.ANYGPU_OK
    assert bool((out == 6.0).all())                      # capture launches nothing
    other_q, other_k, other_v = _operands(4, 2, 2, 900, 64, 80)
    other = torch.empty_like(other_q)
    for replay in range(3):
        out.fill_(float(replay))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"
        # the library's own eager work between the replays, through the same array
        assert f(other_q.data_ptr(), other_k.data_ptr(), other_v.data_ptr(), other.data_ptr(), 4, 2, 2, 900, 64, 0.125, 0.0, 1, 0,
                 None) == capi.ANYGPU_OK
        torch.cuda.synchronize()
    # (the graph object itself holds a little memory of the runtime's; the library's 64 MiB workspace would show)
    assert free_before - torch.cuda.mem_get_info()[0] < 16 * GRANULE
