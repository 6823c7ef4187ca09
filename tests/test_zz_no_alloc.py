"""GPU test of trn_attn_fwd_noalloc_f16, the entry point that allocates nothing: its split-key workspace is a static
device array inside the library.  Called through the C ABI and held to the existing entry point with a caller-provided
workspace (trn_attn_fwd_ws_f16): same kernel, same share order, so the fp16 outputs and fp32 row normalisers must be
bit-identical; and to the CPU oracle at the usual tolerance (fp16 outputs atol 2e-2 / rtol 1e-2, log-sum-exp 1e-3).
Two calls in a row, the second on a smaller problem, so that whatever the first left in the array is there to hurt."""
import ctypes as C

import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def _problem(B, Hq, Hkv, Sq, Skv, D, seed):
    g = torch.Generator().manual_seed(seed)
    return (ref.randn_half((B, Hq, Sq, D), g), ref.randn_half((B, Hkv, Skv, D), g), ref.randn_half((B, Hkv, Skv, D), g))


def _run_both(shape, causal, seed):
    from triton_amd import _lib, ops
    B, Hq, Hkv, Sq, Skv, D = shape
    q, k, v = _problem(*shape, seed)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o_ws = torch.zeros_like(qd); lse_ws = torch.zeros(B, Hq, Sq, device="cuda")
    o_st = torch.zeros_like(qd); lse_st = torch.zeros(B, Hq, Sq, device="cuda")
    need = ops.attention_workspace_bytes(qd, kd, vd, o_ws, scale, causal)
    assert 0 < need <= 8 << 20, "the shape is meant to take the split path within the static array"
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    ops.attention(qd, kd, vd, o_ws, scale, causal, lse=lse_ws, workspace=ws)
    # straight through the C ABI, no Python-side helper deciding anything
    lib = _lib.load()
    d = ops._attn_desc(qd, kd, vd, o_st, scale, causal, False, 0.0, None, 1.0)
    st = lib.trn_attn_fwd_noalloc_f16(C.byref(d), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o_st.data_ptr(),
                                      lse_st.data_ptr(), None, None, None, torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.trn_status_name(st)
    torch.cuda.synchronize()
    assert torch.equal(o_st, o_ws) and torch.equal(lse_st, lse_ws)
    want, want_lse = ref.attention(q, k, v, scale, causal, return_lse=True)
    assert torch.allclose(o_st.float().cpu(), want.float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(lse_st.cpu(), want_lse, atol=1e-3, rtol=1e-3)


def test_static_scratch_matches_caller_workspace_twice_second_smaller():
    from triton_amd import _lib
    assert _lib.load().trn_check_device() == 0
    _run_both((1, 32, 8, 16, 8208, 128), True, seed=11)     # 32 heads x 8 shares
    _run_both((1, 8, 2, 5, 4200, 128), False, seed=12)      # fewer heads, fewer keys, other share count


def test_static_scratch_many_heads_two_shares_and_shapes_that_need_none():
    from triton_amd import _lib, ops
    lib = _lib.load()
    # 120 heads (GQA 15:1), two shares each: the largest head count that still splits
    _run_both((1, 120, 8, 4, 8192, 128), False, seed=13)
    assert lib.trn_status_name(-8) == b"TRN_E_SCRATCH"
    # a prefill shape uses no scratch: same as trn_attn_fwd_f16
    g = torch.Generator().manual_seed(5)
    q2 = ref.randn_half((1, 4, 128, 64), g); k2 = ref.randn_half((1, 2, 128, 64), g); v2 = ref.randn_half((1, 2, 128, 64), g)
    qd, kd, vd = q2.cuda(), k2.cuda(), v2.cuda(); o2 = torch.zeros_like(qd); o3 = torch.zeros_like(qd)
    d2 = ops._attn_desc(qd, kd, vd, o2, 0.125, True, False, 0.0, None, 1.0)
    st = lib.trn_attn_fwd_noalloc_f16(C.byref(d2), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o2.data_ptr(), None, None,
                                      None, None, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    ops.attention(qd, kd, vd, o3, 0.125, True)
    torch.cuda.synchronize()
    assert torch.equal(o2, o3)


def test_static_scratch_call_captured_into_a_graph_and_replayed():
    """The entry point is meant for code under graph capture: captured once (after the eager call above has looked up
    the array's address), replayed with the program's own eager work and synchronisations between the replays, every
    replay held to the eager result bit for bit -- on fresh inputs each time, so a replay that did nothing would show."""
    from triton_amd import ops
    B, Hq, Hkv, Sq, Skv, D = 1, 32, 8, 16, 8208, 128
    q, k, v = _problem(B, Hq, Hkv, Sq, Skv, D, seed=21)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o_g = torch.zeros_like(qd); lse_g = torch.zeros(B, Hq, Sq, device="cuda")
    o_e = torch.zeros_like(qd); lse_e = torch.zeros(B, Hq, Sq, device="cuda")
    assert ops.attention_workspace_bytes(qd, kd, vd, o_g, scale, True) > 0
    ops.attention(qd, kd, vd, o_e, scale, True, lse=lse_e, workspace="static")     # eager first: address looked up here
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            ops.attention(qd, kd, vd, o_g, scale, True, lse=lse_g, workspace="static")
    stream.synchronize()
    gen = torch.Generator().manual_seed(22)
    for rep in range(3):
        qd.copy_(ref.randn_half(tuple(q.shape), gen)); kd.copy_(ref.randn_half(tuple(k.shape), gen))
        o_g.zero_(); lse_g.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            graph.replay()
        stream.synchronize()
        ops.attention(qd, kd, vd, o_e, scale, True, lse=lse_e, workspace="static")
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(lse_g, lse_e), f"replay {rep}"
    want, want_lse = ref.attention(qd.cpu(), kd.cpu(), vd.cpu(), scale, True, return_lse=True)
    assert torch.allclose(o_g.float().cpu(), want.float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(lse_g.cpu(), want_lse, atol=1e-3, rtol=1e-3)
