"""GPU parity for trn_attn_fwd_ws_f16: decode shapes (at most 32 queries per head) whose keys are split over several
workgroups through a caller-provided workspace.  Checked against the CPU oracle (fp16 outputs atol 2e-2 / rtol 1e-2,
fp32 log-sum-exp 1e-3) and against the entry point without a workspace."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def close(got, want, atol=2e-2, rtol=1e-2):
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), f"{int(bad.sum())} elements off; max abs err {err.max():.4g}"


def make(B, Hq, Hkv, Sq, Skv, D, seed=7):
    g = torch.Generator().manual_seed(seed)
    return (ref.randn_half((B, Hq, Sq, D), g), ref.randn_half((B, Hkv, Skv, D), g), ref.randn_half((B, Hkv, Skv, D), g))


def workspace_for(q, k, v, o, scale, causal):
    from triton_amd import ops
    n = ops.attention_workspace_bytes(q, k, v, o, scale, causal)
    return n, (torch.zeros(n, dtype=torch.uint8, device="cuda") if n else None)


SPLIT_CASES = [
    # B, Hq, Hkv, Sq, Skv, D, causal
    (1, 32, 32, 16, 8208, 128, False),   # eight times the reference's decode-append cache at Llama widths
    (1, 32, 8, 16, 8200, 128, True),     # GQA, causal with a cached prefix
    (1, 71, 1, 16, 8300, 64, False),     # Falcon: MQA, 71 heads of width 64
    (2, 4, 2, 1, 4099, 128, True),       # one query, ragged keys, many shares
    (1, 3, 1, 32, 4129, 128, True),      # 130 blocks in shares of 9: the last share is short
    (1, 8, 8, 7, 20000, 128, False),     # long cache
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal", SPLIT_CASES)
def test_split_keys_match_oracle_and_unsplit(B, Hq, Hkv, Sq, Skv, D, causal):
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); o1 = torch.zeros_like(qd)
    lse = torch.zeros(B, Hq, Sq, device="cuda"); lse1 = torch.zeros_like(lse)
    n, ws = workspace_for(qd, kd, vd, o, scale, causal)
    assert n > 0, "this shape is meant to take the split path"
    # the arrival counters are left at zero, so repeated calls need no clearing; the earlier calls see other keys and
    # values, so shares left in the workspace by them would show in the last call's result
    for kk, vv in ((kd.flip(2), vd.flip(2)), (vd, kd), (kd, vd)):
        o.zero_()
        ops.attention(qd, kk.contiguous(), vv.contiguous(), o, scale, causal, lse=lse, workspace=ws)
    ops.attention(qd, kd, vd, o1, scale, causal, lse=lse1)
    torch.cuda.synchronize()
    want, want_lse = ref.attention(q, k, v, scale, causal, return_lse=True)
    close(o, want); close(lse, want_lse, atol=1e-3, rtol=1e-3)
    close(o, o1, atol=2e-3, rtol=2e-3); close(lse, lse1, atol=1e-4, rtol=1e-5)
    counters = ws[:((B * Hq + 63) // 64) * 256].view(torch.int32)
    assert int(counters.abs().sum()) == 0


def test_split_keys_with_noise_and_fused_q_norm():
    from triton_amd import ops
    B, Hq, Hkv, Sq, Skv, D = 1, 8, 2, 16, 4112, 128
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=3)
    noise = ref.gumbel_noise((B, Hq, Sq, Skv), 99)
    tau, scale = 1.5, D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda"); lsep = torch.zeros_like(lse)
    n, ws = workspace_for(qd, kd, vd, o, scale, False)
    assert n > 0
    ops.attention(qd, kd, vd, o, scale, False, lse=lse, noise=noise.cuda(), tau=tau, lse_pert=lsep, workspace=ws)
    torch.cuda.synchronize()
    close(o, ref.attention(q, k, v, scale, False))
    s = ref.scores_fp32(q, k, scale, False)
    close(lsep, torch.logsumexp((s + noise) / tau, -1), atol=1e-3, rtol=1e-3)
    close(lse, torch.logsumexp(s, -1), atol=1e-3, rtol=1e-3)
    # per-head RMSNorm of the queries fused into the kernel (no weight, no eps), as the QKNorm decode module uses it
    gq = torch.ones(D, dtype=torch.float16)
    o.zero_()
    ops.attention(qd, kd, vd, o, scale, False, q_norm=True, gamma_q=None, q_eps=0.0, workspace=ws)
    torch.cuda.synchronize()
    qn = ref.rmsnorm(q, gq, 0.0)
    close(o, ref.attention(qn, k, v, scale, False))


def test_workspace_rules():
    from triton_amd import ops, _lib
    q, k, v = make(1, 8, 8, 16, 4112, 128)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd)
    scale = 128 ** -0.5
    n, ws = workspace_for(qd, kd, vd, o, scale, False)
    want = ref.attention(q, k, v, scale, False)
    # too small a workspace: the call falls back to one workgroup per head and leaves the workspace alone
    small = torch.full((n - 256,), 0x5a, dtype=torch.uint8, device="cuda")
    ops.attention(qd, kd, vd, o, scale, False, workspace=small)
    torch.cuda.synchronize()
    close(o, want); assert bool((small == 0x5a).all())
    # misaligned workspace
    big = torch.zeros(n + 256, dtype=torch.uint8, device="cuda")
    with pytest.raises(_lib.TrnError) as e:
        ops.attention(qd, kd, vd, o, scale, False, workspace=big[16:16 + n])
    assert e.value.status_name == "TRN_E_ALIGN"
    # shapes that do not split report 0 bytes: many heads, too few keys for the head count, or more than 32 queries
    for shape in ((1, 128, 1, 16, 8208, 128), (1, 8, 8, 16, 1040, 128), (1, 8, 8, 16, 4080, 128), (1, 32, 8, 16, 4112, 128),
                  (1, 8, 8, 33, 4112, 128)):
        qq, kk, vv = (t.cuda() for t in make(*shape))
        assert ops.attention_workspace_bytes(qq, kk, vv, torch.zeros_like(qq), scale, False) == 0
    # a workspace handed to a shape that does not use one is ignored
    qq, kk, vv = make(1, 4, 2, 64, 128, 128)
    oo = torch.zeros_like(qq).cuda()
    ops.attention(qq.cuda(), kk.cuda(), vv.cuda(), oo, scale, True, workspace=ws)
    torch.cuda.synchronize()
    close(oo, ref.attention(qq, kk, vv, scale, True))


def test_split_keys_under_graph_replay():
    """Captured once, replayed with eager work between the replays: every replay gives the eager result."""
    from triton_amd import ops
    B, Hq, Hkv, Sq, Skv, D = 1, 32, 8, 16, 8208, 128
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=17)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); o_eager = torch.zeros_like(qd)
    n, ws = workspace_for(qd, kd, vd, o, scale, False)
    ops.attention(qd, kd, vd, o_eager, scale, False, workspace=ws)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        ops.attention(qd, kd, vd, o, scale, False, workspace=ws)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            ops.attention(qd, kd, vd, o, scale, False, workspace=ws)
    stream.synchronize()
    for i in range(4):
        o.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            graph.replay()
        stream.synchronize()
        assert torch.equal(o, o_eager), f"replay {i}"
        kd2 = kd.clone(); torch.cuda.synchronize()          # eager work between replays
        del kd2


def test_decode_modules_split_path_matches_reference_classes():
    """The decode-append modules at a shape where the attention splits its keys (8 heads, 4112 keys); RoCo asks for
    the key statistics, which are a second sweep of the one workgroup per head, so it is not split."""
    from triton_amd import modules
    M, N, D, P = 16, 1024, 128, 4096
    H = N // D
    g = torch.Generator().manual_seed(5)
    cpu = dict(X=ref.reference_recipe((M, N), g) * 30, WQ=ref.reference_recipe((N, N), g) * 30,
               WK=ref.reference_recipe((N, N), g) * 30, WV=ref.reference_recipe((N, N), g) * 30,
               K_cache=ref.reference_recipe((H, P + M, D), g) * 30, V_cache=ref.reference_recipe((H, P + M, D), g) * 30)
    cpu = {k: v.half() for k, v in cpu.items()}
    W = (cpu["WQ"], cpu["WK"], cpu["WV"])
    for variant in ("vanilla", "roco"):
        t = {k: v.cuda() for k, v in cpu.items()}
        t["O2"] = torch.zeros(M, N, dtype=torch.float16, device="cuda")
        t["C_out1"] = torch.zeros(H, P + M, device="cuda"); t["C_out2"] = torch.zeros_like(t["C_out1"])
        mod = modules.get(variant, "decode", head_dim=D)
        for _ in range(2):
            mod.forward(*[t[n] for n in mod.TENSOR_PARAMS])
        torch.cuda.synchronize()
        if variant == "vanilla":
            assert any(k[0] == "attn_ws" for k in mod._ws), "expected the split path"
            want = ref.decode_append_vanilla(cpu["X"], *W, cpu["K_cache"], cpu["V_cache"], P, D)
            close(t["O2"], ref.flatten_token_major(want))
        else:
            wo, s1, s2 = ref.decode_append_roco(cpu["X"], *W, cpu["K_cache"], cpu["V_cache"], P, D)
            close(t["O2"], ref.flatten_token_major(wo))
            # (q, k come from an fp16-rounded GEMM whose summation order differs from the oracle's: 5e-3 relative)
            close(t["C_out1"], s1, atol=1e-6, rtol=5e-3); close(t["C_out2"], s2, atol=1e-8, rtol=5e-3)


# ---- trn_attn_fwd_stats_ws_f16: few heads on a long cache, keys split over workgroups, the statistics as a second launch
STATS_SPLIT_CASES = [
    # B, Hq, Hkv, Sq, Skv, D, causal, with_noise
    (1, 8, 8, 16, 8208, 128, True, False), (1, 8, 2, 16, 8208, 128, False, True), (1, 16, 4, 5, 8200, 64, True, True),
    (1, 32, 8, 16, 16400, 64, True, False), (2, 3, 3, 32, 6147, 128, False, True), (1, 12, 12, 1, 9000, 64, True, False)]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal,with_noise", STATS_SPLIT_CASES)
def test_statistics_with_split_keys_match_oracle_and_single_launch(B, Hq, Hkv, Sq, Skv, D, causal, with_noise):
    """RoCo's sums / KeyFormer's key scores over a long cache: the oracle at 1e-3 relative, and the single-launch form
    of the same call (whose second sweep runs inside the attention kernel) to a tenth of that."""
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=23)
    scale, tau = D ** -0.5, 1.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    n = ops.attention_stats_workspace_bytes(qd, kd, vd, torch.zeros_like(qd), scale, causal)
    assert n > 0 and n == ops.attention_workspace_bytes(qd, kd, vd, torch.zeros_like(qd), scale, causal)
    ws = torch.zeros(n, dtype=torch.uint8, device="cuda")
    pitch = (Skv + 3) // 4 * 4
    noise = None
    if with_noise:
        buf = torch.full((B, Hq, Sq, pitch), float("nan"))
        buf[..., :Skv] = torch.randn(B, Hq, Sq, Skv, generator=torch.Generator().manual_seed(3))
        noise = buf.cuda()[..., :Skv]
    outs = []
    for w in (ws, None):
        o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda"); lsep = torch.zeros_like(lse)
        s1 = torch.full((B, Hq, Skv), -1.0, device="cuda"); s2 = torch.full((B, Hq, Skv), -1.0, device="cuda")
        kw = dict(noise=noise, tau=tau, lse_pert=lsep) if with_noise else {}
        for _ in range(2):          # twice: the second call finds what the first left in the workspace
            ops.attention_with_stats(qd, kd, vd, o, scale, causal, s1, None if with_noise else s2, lse=lse, workspace=w, **kw)
        torch.cuda.synchronize()
        outs.append((o, s1, s2, lse, lsep))
    (o, s1, s2, lse, lsep), (o1, t1, t2, _, _) = outs
    if with_noise:
        wo, wscore = ref.keyformer(q, k, v, noise.cpu(), scale, tau, causal)
        err = (s1.cpu() - wscore).abs()
        assert (err <= 1e-9 + 1e-3 * wscore.abs()).all()
    else:
        wo, w1, w2 = ref.roco(q, k, v, scale, causal)
        assert ((s1.cpu() - w1).abs() <= 1e-9 + 1e-3 * w1.abs()).all() and ((s2.cpu() - w2).abs() <= 1e-9 + 1e-3 * w2.abs()).all()
        close(s2, t2, atol=1e-12, rtol=2e-4)
    close(o, wo); close(o, o1, atol=2e-3, rtol=2e-3)
    close(s1, t1, atol=1e-12, rtol=1e-4)


def test_statistics_workspace_rule_and_fallbacks():
    """Many heads fill the chip by themselves, short caches are launch-bound: no split there, and the entry point with
    a workspace is then the plain one bit for bit; so it is with a workspace that is too small or without the buffer
    for the row normalisers."""
    from triton_amd import ops
    scale = 0.125
    for (B, Hq, Hkv, Sq, Skv, D), want_split in (((1, 71, 1, 16, 16400, 64), False), ((1, 32, 8, 16, 16400, 128), False),
                                                  ((1, 8, 8, 16, 4112, 128), False), ((1, 8, 8, 33, 8208, 128), False),
                                                  ((1, 8, 8, 16, 8208, 128), True), ((1, 16, 16, 4, 8208, 64), True)):
        q = torch.zeros(B, Hq, Sq, D, dtype=torch.float16, device="cuda"); k = torch.zeros(B, Hkv, Skv, D, dtype=torch.float16, device="cuda")
        assert (ops.attention_stats_workspace_bytes(q, k, k, q, scale, True) > 0) == want_split, (Hq, Skv)
    q, k, v = make(1, 8, 8, 16, 8208, 128, seed=29)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    n = ops.attention_stats_workspace_bytes(qd, kd, vd, qd, scale, True)
    assert n > 0
    res = []
    for ws, with_lse in ((None, True), (torch.zeros(n // 2 // 256 * 256, dtype=torch.uint8, device="cuda"), True),
                         (torch.zeros(n, dtype=torch.uint8, device="cuda"), False)):
        o = torch.zeros_like(qd); s1 = torch.zeros(1, 8, 8208, device="cuda"); lse = torch.zeros(1, 8, 16, device="cuda")
        ops.attention_with_stats(qd, kd, vd, o, scale, True, s1, None, lse=lse if with_lse else None, workspace=ws)
        torch.cuda.synchronize()
        res.append((o, s1))
    for o, s1 in res[1:]:
        assert torch.equal(o, res[0][0]) and torch.equal(s1, res[0][1])
