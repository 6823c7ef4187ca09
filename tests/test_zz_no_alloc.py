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
    _run_both((1, 32, 8, 16, 4112, 128), True, seed=11)     # 32 heads x 8 shares
    _run_both((1, 8, 2, 5, 1600, 128), False, seed=12)      # fewer heads, fewer keys, other share count


def test_static_scratch_limit_and_shapes_that_need_none():
    from triton_amd import _lib, ops
    lib = _lib.load()
    # The library shares a head's keys out over at most 256 workgroups in all, so today's largest workspace
    # (256 shares x 32 x (128 + 4) floats + counters = 4.3 MB) fits the 8 MiB array; whatever the policy, a need beyond
    # the array must come back as TRN_E_SCRATCH (-8) and never run.
    B, Hq, Hkv, Sq, Skv, D = 1, 120, 120, 4, 8192, 128
    q = torch.zeros(B, Hq, Sq, D, dtype=torch.float16, device="cuda")
    k = torch.zeros(B, Hkv, Skv, D, dtype=torch.float16, device="cuda"); o = torch.zeros_like(q)
    need = ops.attention_workspace_bytes(q, k, k, o, 1.0, False)
    d = ops._attn_desc(q, k, k, o, 1.0, False, False, 0.0, None, 1.0)
    st = lib.trn_attn_fwd_noalloc_f16(C.byref(d), q.data_ptr(), k.data_ptr(), k.data_ptr(), o.data_ptr(), None, None,
                                      None, None, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert st == (0 if need <= 8 << 20 else -8)
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
