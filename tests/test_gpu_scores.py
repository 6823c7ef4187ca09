"""GPU parity for the key-score paths: forward (row LSE) + trn_attn_colstats_f16, against the CPU oracle.
fp32 key scores: 1e-3 relative.  The absolute allowance is 1e-9: sums of squares of late keys are of order 1e-6 and
below, and a larger allowance would leave exactly those columns unchecked."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def close_scores(got, want, rtol=1e-3, atol=1e-9):
    got = got.float().cpu(); want = want.float()
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), f"{int(bad.sum())} off; max rel {(err / want.abs().clamp(min=1e-6)).max():.3g}"


def make(B, Hq, Hkv, Sq, Skv, D, seed=42):
    g = torch.Generator().manual_seed(seed)
    return (ref.randn_half((B, Hq, Sq, D), g), ref.randn_half((B, Hkv, Skv, D), g), ref.randn_half((B, Hkv, Skv, D), g))


def run_roco(q, k, v, scale, causal):
    from triton_amd import ops
    B, Hq, Sq, D = q.shape; Skv = k.shape[2]
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda")
    s1 = torch.full((B, Hq, Skv), -1.0, device="cuda"); s2 = torch.full((B, Hq, Skv), -1.0, device="cuda")
    ops.attention(qd, kd, vd, o, scale, causal, lse=lse)
    ops.attention_colstats(qd, kd, lse, scale, causal, s1, s2)
    torch.cuda.synchronize()
    return o, s1, s2


CASES = [(1, 4, 2, 256, 256, 128, True), (1, 4, 2, 256, 256, 128, False), (2, 3, 1, 200, 200, 64, True),
         (1, 2, 2, 16, 1040, 128, False), (1, 2, 2, 16, 1040, 64, True), (1, 8, 2, 640, 640, 128, True),
         (1, 1, 1, 1, 1, 64, True), (1, 2, 1, 130, 259, 128, True),
         # longer walks of the statistics pass: several mask-free turns of its stage ring, key tiles in pairs with a
         # middle one left over, more queries than keys without a mask, a long cached prefix under the mask
         (1, 1, 1, 1024, 1024, 128, True), (1, 2, 1, 700, 300, 128, False), (1, 2, 2, 520, 1000, 64, True),
         (1, 2, 1, 1100, 1100, 64, True)]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal", CASES)
def test_roco_parity(B, Hq, Hkv, Sq, Skv, D, causal):
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D)
    scale = D ** -0.5
    o, s1, s2 = run_roco(q, k, v, scale, causal)
    wo, w1, w2 = ref.roco(q, k, v, scale, causal)
    close_scores(s1, w1); close_scores(s2, w2)
    assert (o.float().cpu() - wo.float()).abs().max() < 2e-2
    # invariant: every row sums to 1, so the column sums add up to the number of queries
    assert torch.allclose(s1.sum(-1).cpu(), torch.full((B, Hq), float(Sq)), rtol=1e-4)


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal,tau", [
    (1, 4, 2, 256, 256, 128, True, 1.0), (1, 4, 2, 200, 200, 128, True, 1.5), (1, 3, 1, 96, 96, 64, False, 1.0),
    (1, 2, 2, 16, 1040, 128, False, 1.5), (1, 2, 1, 130, 260, 64, True, 1.0),
    (2, 4, 2, 9, 700, 128, True, 1.5), (1, 3, 1, 32, 100, 64, True, 1.0),     # decode kernel with noise, GQA / MQA
    # longer walks of both passes: several turns of the statistics pass's stage ring, a cached prefix, both widths
    (1, 2, 1, 600, 600, 64, True, 1.0), (1, 2, 2, 520, 1000, 128, True, 1.5), (1, 2, 1, 700, 300, 64, False, 1.0)])
def test_keyformer_parity(B, Hq, Hkv, Sq, Skv, D, causal, tau):
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=7)
    noise = ref.gumbel_noise((B, Hq, Sq, Skv), 1234)
    scale = D ** -0.5
    qd, kd, vd, nd = q.cuda(), k.cuda(), v.cuda(), noise.cuda()
    o = torch.zeros_like(qd); lsep = torch.zeros(B, Hq, Sq, device="cuda")
    score = torch.full((B, Hq, Skv), -1.0, device="cuda")
    ops.attention(qd, kd, vd, o, scale, causal, noise=nd, tau=tau, lse_pert=lsep)
    ops.attention_colstats(qd, kd, lsep, scale, causal, score, None, noise=nd, tau=tau)
    torch.cuda.synchronize()
    wo, wscore = ref.keyformer(q, k, v, noise, scale, tau, causal)
    close_scores(score, wscore)
    assert (o.float().cpu() - wo.float()).abs().max() < 2e-2
    assert torch.allclose(score.sum(-1).cpu(), torch.full((B, Hq), float(Sq)), rtol=1e-4)


def _nan_padded(noise):
    """fp32 device copy of `noise` whose rows are padded to a multiple of 4 floats, the padding filled with NaN."""
    B, H, Sq, Skv = noise.shape
    buf = torch.full((B, H, Sq, (Skv + 3) // 4 * 4), float("nan"), device="cuda")
    view = buf[..., :Skv]
    view.copy_(noise)
    return view


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal,tau", [
    (1, 2, 1, 130, 257, 64, True, 1.0), (1, 2, 2, 203, 203, 128, True, 1.5), (1, 3, 1, 70, 198, 128, False, 1.0),   # prefill kernels
    (1, 4, 2, 16, 1041, 128, False, 1.5), (2, 2, 2, 9, 702, 64, True, 1.0), (1, 3, 1, 32, 99, 128, True, 1.0)])     # decode kernel
def test_keyformer_any_key_count_padding_never_read(B, Hq, Hkv, Sq, Skv, D, causal, tau):
    """The reference's KeyFormer takes any cache length (ref_rms.py:147-179).  The kernels fetch noise 16 bytes at a
    time, so its rows are padded to 4 floats; whatever the padding holds (NaN here) must never reach a sum."""
    from triton_amd import ops
    assert Skv % 4 != 0
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=21)
    noise = ref.gumbel_noise((B, Hq, Sq, Skv), 77)
    scale = D ** -0.5
    qd, kd, vd, nd = q.cuda(), k.cuda(), v.cuda(), _nan_padded(noise)
    o = torch.zeros_like(qd); lsep = torch.zeros(B, Hq, Sq, device="cuda"); score = torch.full((B, Hq, Skv), -1.0, device="cuda")
    ops.attention_with_stats(qd, kd, vd, o, scale, causal, score, None, noise=nd, tau=tau, lse_pert=lsep)
    torch.cuda.synchronize()
    wo, wscore = ref.keyformer(q, k, v, noise, scale, tau, causal)
    close_scores(score, wscore)
    assert (o.float().cpu() - wo.float()).abs().max() < 2e-2
    s = ref.scores_fp32(q, k, scale, causal)
    assert torch.allclose(lsep.cpu(), torch.logsumexp((s + noise) / tau, -1), atol=1e-3, rtol=1e-3)


def test_keyformer_split_keys_any_key_count():
    from triton_amd import ops
    B, Hq, Hkv, Sq, Skv, D, tau = 1, 8, 2, 16, 4115, 128, 1.5
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=22)
    noise = ref.gumbel_noise((B, Hq, Sq, Skv), 78)
    scale = D ** -0.5
    qd, kd, vd, nd = q.cuda(), k.cuda(), v.cuda(), _nan_padded(noise)
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda"); lsep = torch.zeros_like(lse)
    n = ops.attention_workspace_bytes(qd, kd, vd, o, scale, False)
    assert n > 0
    ws = torch.zeros(n, dtype=torch.uint8, device="cuda")
    ops.attention(qd, kd, vd, o, scale, False, lse=lse, noise=nd, tau=tau, lse_pert=lsep, workspace=ws)
    torch.cuda.synchronize()
    s = ref.scores_fp32(q, k, scale, False)
    assert torch.allclose(lsep.cpu(), torch.logsumexp((s + noise) / tau, -1), atol=1e-3, rtol=1e-3)
    assert (o.float().cpu() - ref.attention(q, k, v, scale, False).float()).abs().max() < 2e-2


@pytest.mark.parametrize("form,PM", [("decode", 1041), ("decode", 1042), ("prefill", 203)])
def test_keyformer_modules_take_fp16_noise_of_any_length(form, PM):
    """Through the module protocol with the reference's fp16 noise (convert_eval_rms.py:201) and a cache length that
    is not a multiple of 4: the module pads its fp32 copy."""
    from triton_amd import modules
    g = torch.Generator().manual_seed(31)
    if form == "decode":
        M, N, D, H = 16, 512, 128, 4
        P = PM - M
        rnd = lambda *sh: (torch.randn(*sh, generator=g).clamp(-1, 1) * 0.05).half()
        X, WQ, WK, WV = rnd(M, N), rnd(N, N), rnd(N, N), rnd(N, N)
        Kc, Vc = rnd(H, PM, D), rnd(H, PM, D)
        noise = torch.randn(H, M, PM, generator=g).half()
        t = dict(X=X.cuda(), WQ=WQ.cuda(), WK=WK.cuda(), WV=WV.cuda(), K_cache=Kc.cuda(), V_cache=Vc.cuda(),
                 O2=torch.zeros(M, N, dtype=torch.float16, device="cuda"), noise=noise.cuda(),
                 C_out=torch.zeros(H, PM, dtype=torch.float16, device="cuda"))
        m = modules.get("keyformer", "decode", head_dim=D)
        m.forward(*[t[p] for p in m.TENSOR_PARAMS])
        torch.cuda.synchronize()
        wo, pw = ref.decode_append_keyformer(X, WQ, WK, WV, Kc, Vc, noise.float(), P, D, tau=1.5)
        assert torch.allclose(t["O2"].float().cpu(), ref.flatten_token_major(wo).float(), atol=2e-2, rtol=1e-2)
        close_scores(t["C_out"], pw.sum(1), rtol=2e-3, atol=1e-3)     # fp16 C_out: its own rounding on top of 1e-3
    else:
        B, Hq, Hkv, S, D = 1, 4, 2, PM, 64
        q, k, v = make(B, Hq, Hkv, S, S, D, seed=32)
        noise = ref.gumbel_noise((B, Hq, S, S), 79).half()
        C_out = torch.zeros(B, Hq, S, device="cuda"); O = torch.zeros(B, Hq, S, D, dtype=torch.float16, device="cuda")
        m = modules.get("keyformer", tau=1.0)
        t = dict(Q=q.cuda(), K=k.cuda(), V=v.cuda(), O=O, noise=noise.cuda(), C_out=C_out)
        m.forward(*[t[p] for p in m.TENSOR_PARAMS])
        torch.cuda.synchronize()
        wo, wc = ref.keyformer(q, k, v, noise.float(), D ** -0.5, 1.0, True)
        close_scores(C_out, wc)
        assert (O.float().cpu() - wo.float()).abs().max() < 2e-2


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal", [(1, 2, 1, 40, 40, 64, True), (2, 4, 2, 33, 70, 128, True),
                                                      (1, 3, 3, 50, 50, 64, False), (1, 2, 2, 130, 259, 128, True)])
def test_roco_mean_and_std_from_the_kernel_against_numpy(B, Hq, Hkv, Sq, Skv, D, causal):
    """trn_attn_colmeanstd_f16: per-key mean and standard deviation of the probabilities over the queries that see
    the key, held to numpy's mean / std (population) of exactly those entries of the fp64 probability matrix."""
    import numpy as np
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=13)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda")
    mean = torch.full((B, Hq, Skv), -1.0, device="cuda"); std = torch.full((B, Hq, Skv), -1.0, device="cuda")
    ops.attention(qd, kd, vd, o, scale, causal, lse=lse)
    ops.attention_col_mean_std(qd, kd, lse, scale, causal, mean, std)
    torch.cuda.synchronize()
    p = torch.softmax(ref.scores_fp32(q, k, scale, causal).double(), -1).numpy()
    off = Skv - Sq
    wm = np.zeros((B, Hq, Skv)); ws = np.zeros((B, Hq, Skv))
    for j in range(Skv):
        first = max(0, j - off) if causal else 0              # first query that sees key j
        col = p[:, :, first:, j]
        wm[:, :, j] = col.mean(-1); ws[:, :, j] = col.std(-1)
    close_scores(mean, torch.from_numpy(wm), rtol=1e-3, atol=1e-7)
    # sqrt(E p^2 - mean^2) in fp32 loses digits where the spread is far below the mean; such keys are held to 1e-3
    # of the mean instead
    err = (std.double().cpu() - torch.from_numpy(ws)).abs()
    assert (err <= 2e-3 * torch.from_numpy(ws) + 1e-3 * torch.from_numpy(wm) + 1e-7).all()


def test_uniform_attention_harmonic_closed_form_on_gpu():
    S, D = 300, 128
    q, k, v = make(1, 2, 1, S, S, D, seed=3)
    o, s1, s2 = run_roco(torch.zeros_like(q), k, v, 1.0, True)
    want1 = ref.harmonic_tail(S, 1).float(); want2 = ref.harmonic_tail(S, 2).float()
    close_scores(s1[0, 0], want1, rtol=1e-4); close_scores(s2[0, 1], want2, rtol=1e-4)


def test_colstats_deterministic():
    q, k, v = make(1, 4, 2, 384, 384, 128, seed=5)
    _, a1, a2 = run_roco(q, k, v, 0.088, True)
    _, b1, b2 = run_roco(q, k, v, 0.088, True)
    assert torch.equal(a1, b1) and torch.equal(a2, b2)


# ---- trn_attn_fwd_stats_f16: attention + statistics in one call (one launch with at most 32 queries per head)
FUSED = [(1, 4, 4, 16, 1040, 128, False), (1, 4, 2, 16, 1040, 128, True), (2, 6, 1, 7, 333, 64, True),
         (1, 3, 3, 32, 32, 128, True), (1, 2, 2, 1, 100, 64, False), (1, 71, 1, 16, 1040, 64, False),
         (1, 4, 2, 130, 259, 128, True)]                     # more than 32 queries: two launches inside the call


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal", FUSED)
def test_fused_attention_and_roco_statistics(B, Hq, Hkv, Sq, Skv, D, causal):
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=11)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda")
    s1 = torch.full((B, Hq, Skv), -1.0, device="cuda"); s2 = torch.full((B, Hq, Skv), -1.0, device="cuda")
    ops.attention_with_stats(qd, kd, vd, o, scale, causal, s1, s2, lse=lse)
    torch.cuda.synchronize()
    wo, w1, w2 = ref.roco(q, k, v, scale, causal)
    close_scores(s1, w1); close_scores(s2, w2)
    assert (o.float().cpu() - wo.float()).abs().max() < 2e-2
    assert torch.allclose(s1.sum(-1).cpu(), torch.full((B, Hq), float(Sq)), rtol=1e-4)
    # the same numbers as the two separate calls (within summation order)
    o2, t1, t2 = run_roco(q, k, v, scale, causal)
    close_scores(s1, t1.cpu(), rtol=1e-4); close_scores(s2, t2.cpu(), rtol=1e-4)
    # only one of the two statistics
    s1b = torch.full_like(s1, -1.0)
    ops.attention_with_stats(qd, kd, vd, o, scale, causal, s1b, None, lse=lse)
    torch.cuda.synchronize()
    assert torch.equal(s1b, s1)


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal,tau", [(1, 4, 4, 16, 1040, 128, False, 1.5), (2, 4, 2, 9, 700, 128, True, 1.5),
                                                          (1, 3, 1, 32, 100, 64, True, 1.0), (1, 2, 1, 130, 260, 64, True, 1.0)])
def test_fused_attention_and_keyformer_scores(B, Hq, Hkv, Sq, Skv, D, causal, tau):
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=7)
    noise = ref.gumbel_noise((B, Hq, Sq, Skv), 1234)
    scale = D ** -0.5
    o = torch.zeros_like(q).cuda(); lsep = torch.zeros(B, Hq, Sq, device="cuda")
    score = torch.full((B, Hq, Skv), -1.0, device="cuda")
    ops.attention_with_stats(q.cuda(), k.cuda(), v.cuda(), o, scale, causal, score, None, noise=noise.cuda(), tau=tau, lse_pert=lsep)
    torch.cuda.synchronize()
    wo, wscore = ref.keyformer(q, k, v, noise, scale, tau, causal)
    close_scores(score, wscore)
    assert (o.float().cpu() - wo.float()).abs().max() < 2e-2
    assert torch.allclose(score.sum(-1).cpu(), torch.full((B, Hq), float(Sq)), rtol=1e-4)


def test_fused_statistics_argument_rules():
    from triton_amd import ops, _lib
    q, k, v = make(1, 2, 2, 64, 64, 64)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); s1 = torch.zeros(1, 2, 64, device="cuda")
    with pytest.raises(_lib.TrnError) as e:          # more than 32 queries and no buffer for the row normalisers
        ops.attention_with_stats(qd, kd, vd, o, 0.125, True, s1)
    assert e.value.status_name == "TRN_E_NULL"
    with pytest.raises(ValueError):
        ops.attention_with_stats(qd, kd, vd, o, 0.125, True, None, None)


# ---- trn_attn_fwd_stats_half_f16: the same launch with fp16 noise and fp16 statistics (the reference's own tensors)
@pytest.mark.gpu
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal,with_noise", [
    (1, 4, 4, 16, 1040, 128, False, True), (1, 4, 2, 16, 1040, 128, True, False), (2, 6, 1, 7, 332, 64, True, True),
    (1, 71, 1, 16, 1040, 64, False, False), (1, 3, 3, 32, 36, 128, True, True), (1, 2, 2, 1, 100, 64, False, True),
    # odd key counts: the last row's last key sits in a dword that is half padding
    (1, 4, 4, 16, 333, 128, True, True), (1, 2, 1, 16, 1041, 64, False, True), (1, 2, 2, 3, 35, 128, False, True)])
def test_fused_statistics_with_fp16_noise_and_outputs(B, Hq, Hkv, Sq, Skv, D, causal, with_noise):
    """Held to the fp32 form of the same call bit for bit: the fp16 noise widened is the same noise, and an fp16 statistic
    is the fp32 one rounded once.  (The fp32 form is held to the oracle above.)"""
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=17)
    scale, tau = D ** -0.5, 1.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    g = torch.Generator().manual_seed(5)
    pitch = (Skv + 3) // 4 * 4
    n16 = torch.full((B, Hq, Sq, pitch), float("nan"), dtype=torch.float16)
    n16[..., :Skv] = torch.randn(B, Hq, Sq, Skv, generator=g).half()
    n16 = n16.cuda()[..., :Skv] if with_noise else None
    n32 = None
    if with_noise:
        buf = torch.full((B, Hq, Sq, pitch), float("nan"), device="cuda"); buf[..., :Skv] = n16.float(); n32 = buf[..., :Skv]
    o1 = torch.zeros_like(qd); o2 = torch.zeros_like(qd)
    lp1 = torch.zeros(B, Hq, Sq, device="cuda"); lp2 = torch.zeros_like(lp1)
    a1 = torch.full((B, Hq, Skv), -1.0, device="cuda"); a2 = torch.full((B, Hq, Skv), -1.0, device="cuda")
    h1 = torch.full((B, Hq, Skv), -1.0, device="cuda", dtype=torch.float16); h2 = torch.full_like(h1, -1.0)
    kw32 = dict(noise=n32, tau=tau, lse_pert=lp1) if with_noise else dict(lse=lp1)
    kw16 = dict(noise=n16, tau=tau, lse_pert=lp2) if with_noise else dict(lse=lp2)
    ops.attention_with_stats(qd, kd, vd, o1, scale, causal, a1, a2, **kw32)
    ops.attention_with_stats_half(qd, kd, vd, o2, scale, causal, h1, h2, **kw16)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(lp1, lp2)
    assert torch.equal(h1, a1.half()) and torch.equal(h2, a2.half())


@pytest.mark.gpu
def test_fp16_statistics_form_refuses_prefill_shapes():
    from triton_amd import ops
    q, k, v = make(1, 2, 2, 33, 64, 64)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    h1 = torch.zeros(1, 2, 64, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError):
        ops.attention_with_stats_half(qd, kd, vd, torch.zeros_like(qd), 0.125, True, h1)
