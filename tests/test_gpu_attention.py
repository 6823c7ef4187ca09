"""GPU parity: trn_attn_fwd_f16 (through the C ABI) against the CPU oracle.
Tolerance for fp16 attention outputs: atol 2e-2, rtol 1e-2; LSE fp32: 1e-3 relative + 1e-3 abs."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


def close(got, want, atol=ATOL, rtol=RTOL):
    got = got.float().cpu(); want = want.float()
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), f"{int(bad.sum())} elements off; max abs err {err.max():.4g}"
    return err.max().item()


def make(B, Hq, Hkv, Sq, Skv, D, seed=42, std=1.0):
    g = torch.Generator().manual_seed(seed)
    q = ref.randn_half((B, Hq, Sq, D), g, 0, std)
    k = ref.randn_half((B, Hkv, Skv, D), g, 0, std)
    v = ref.randn_half((B, Hkv, Skv, D), g, 0, std)
    return q, k, v


CASES = [
    # B, Hq, Hkv, Sq, Skv, D, causal
    (1, 4, 2, 128, 128, 128, True),
    (1, 4, 2, 128, 128, 128, False),
    (2, 8, 2, 512, 512, 128, True),
    (1, 2, 1, 300, 300, 128, True),      # ragged
    (1, 3, 1, 77, 77, 64, True),         # MQA, D=64, ragged
    (1, 6, 1, 256, 256, 64, True),
    (1, 4, 4, 16, 1040, 128, False),     # the reference's decode-append shape (M=16, P=1024)
    (1, 4, 4, 16, 1040, 128, True),      # causal with a cached prefix
    (1, 5, 5, 16, 1040, 64, False),
    (1, 2, 2, 1, 1, 64, True),
    (1, 2, 1, 129, 257, 128, True),
    (2, 32, 8, 1024, 1024, 128, True),   # enough workgroups for the 8-wave (256-query) tile shape
    (2, 32, 8, 1000, 1000, 128, False),  # the same, ragged
    (1, 72, 1, 1100, 1100, 64, True),
    # at most 32 queries per head: the decode kernel (waves split the keys), GQA / MQA, ragged key counts
    (2, 8, 2, 16, 1040, 128, True),
    (1, 6, 1, 7, 333, 64, True),
    (1, 4, 2, 32, 32, 128, True),
    (3, 4, 4, 32, 5000, 128, False),
    (1, 4, 2, 33, 1040, 128, True),      # one query more: back to the prefill kernel
    # head_dim 128 with one workgroup per head (a single V stage, refilled behind its last reader): too few keys for
    # column shares, and too many heads for them; several blocks per wave, causal and not
    (1, 8, 8, 16, 216, 128, True),
    (1, 8, 2, 16, 64, 128, False),
    (1, 136, 8, 16, 1040, 128, True),
    (2, 80, 80, 5, 2100, 128, False),
    (1, 64, 8, 1990, 2100, 128, True),   # 8-wave workgroups under a causal mask with a cached prefix and ragged ends:
                                         # the waves of a workgroup stop at different tiles
    (1, 16, 16, 520, 520, 64, True),     # head_dim 64 stays on 4-wave workgroups; a last workgroup of 8 queries
    # causal grids of a single round run "paired" (a workgroup's two wave groups own 128-query tiles from opposite
    # ends of the sequence): an odd tile count (the middle tile is alone), ragged ends, a cached prefix, both widths
    (1, 96, 8, 600, 600, 128, True),
    (1, 96, 8, 600, 700, 128, True),
    (2, 64, 64, 500, 500, 64, True),
    (1, 32, 8, 2048, 2048, 128, True),   # the attention of the PreNorm block (the 2048-token PreNorm workload)
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal", CASES)
def test_attention_parity(B, Hq, Hkv, Sq, Skv, D, causal):
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    od = torch.zeros_like(qd)
    lse = torch.zeros(B, Hq, Sq, dtype=torch.float32, device="cuda")
    ops.attention(qd, kd, vd, od, scale, causal, lse=lse)
    torch.cuda.synchronize()
    want, want_lse = ref.attention(q, k, v, scale, causal, return_lse=True)
    close(od, want)
    close(lse, want_lse, atol=1e-3, rtol=1e-3)


def _random_shapes(n, seed):
    import random
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        D = rnd.choice((64, 128))
        Hkv = rnd.choice((1, 2, 3))
        Hq = Hkv * rnd.choice((1, 2, 4))
        B = rnd.choice((1, 2))
        causal = rnd.random() < 0.6
        Sq = rnd.choice((33, 40, 64, 97, 128, 129, 200, 255, 256, 257, 300, 384, 511, 513, 640))
        Skv = Sq + rnd.choice((0, 0, 1, 31, 32, 33, 64, 100, 257)) if causal else rnd.choice((1, 17, 32, 63, 64, 65, 200, 333, 512, 700))
        out.append((B, Hq, Hkv, Sq, Skv, D, causal, rnd.random() < 0.3))
    return out


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal,qnorm", _random_shapes(48, 20260101))
def test_attention_parity_seeded_random_shapes(B, Hq, Hkv, Sq, Skv, D, causal, qnorm):
    """A seeded sweep over ragged query / key counts on both sides of the 32-, 64- and 256-row tile edges, GQA ratios,
    cached prefixes of every alignment, both head widths, with and without the fused query norm."""
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=Sq * 1000 + Skv)
    scale = D ** -0.5
    od = torch.zeros_like(q).cuda()
    lse = torch.zeros(B, Hq, Sq, dtype=torch.float32, device="cuda")
    ops.attention(q.cuda(), k.cuda(), v.cuda(), od, scale, causal, lse=lse, q_norm=qnorm, gamma_q=None, q_eps=0.0)
    torch.cuda.synchronize()
    qq = ref.rmsnorm(q, torch.ones(D, dtype=torch.float16), 0.0) if qnorm else q
    want, want_lse = ref.attention(qq, k, v, scale, causal, return_lse=True)
    close(od, want)
    close(lse, want_lse, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D,causal", [
    (1, 4, 2, 300, 300, 128, True), (1, 4, 4, 256, 520, 64, False), (2, 32, 8, 1024, 1024, 128, True),
    (1, 32, 8, 2048, 2048, 128, True), (1, 8, 1, 700, 700, 64, True), (1, 4, 2, 16, 1040, 128, True)])
def test_attention_scores_that_rise_and_jump_along_the_keys(B, Hq, Hkv, Sq, Skv, D, causal):
    """The kernels keep a lazy reference maximum, set by the first 32-key block and raised only when a later block
    exceeds it by more than 2^8; N(0,1) inputs never get there.  Here the keys grow sevenfold along the sequence, so the
    block maxima climb through several raises, and three late keys are multiples of particular queries, so that single
    scores jump tens of binades above everything before them (a probability formed against the old reference would be
    infinite in fp16).  Outputs and row normalisers against the oracle at the usual tolerances."""
    from triton_amd import ops
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, seed=31)
    k = (k.float() * (1.0 + 6.0 * torch.arange(Skv).float() / Skv)[None, None, :, None]).half()
    G = Hq // Hkv
    for key, qi in ((Skv - 3, Sq - 1), (Skv // 2 + 5, Sq // 2), (40, min(Sq - 1, 45))):     # key j = 3 x query qi of the KV head's first query head
        k[:, :, key] = (3.0 * q[:, ::G, qi].float()).half()
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda")
    ops.attention(qd, kd, vd, o, scale, causal, lse=lse)
    torch.cuda.synchronize()
    want, want_lse = ref.attention(q, k, v, scale, causal, return_lse=True)
    assert torch.isfinite(o).all() and torch.isfinite(lse).all()
    close(o, want)
    close(lse, want_lse, atol=2e-3, rtol=1e-3)


def test_attention_reference_recipe_unscaled():
    """The reference's own input recipe and semantics: scale 1, no mask (ref_rms.py:77-78)."""
    from triton_amd import ops
    g = torch.Generator().manual_seed(42)
    q = ref.reference_recipe((1, 8, 16, 128), g); k = ref.reference_recipe((1, 8, 1040, 128), g)
    v = ref.reference_recipe((1, 8, 1040, 128), g)
    od = torch.zeros_like(q).cuda()
    ops.attention(q.cuda(), k.cuda(), v.cuda(), od, 1.0, False)
    torch.cuda.synchronize()
    close(od, ref.attention(q, k, v, 1.0, False), atol=1e-4, rtol=1e-2)


def test_attention_closed_forms_on_gpu():
    from triton_amd import ops
    q, k, v = make(1, 4, 2, 200, 200, 128, seed=7)
    od = torch.zeros_like(q).cuda()
    ops.attention(torch.zeros_like(q).cuda(), k.cuda(), v.cuda(), od, 0.1, True)
    torch.cuda.synchronize()
    want = (v.float().repeat_interleave(2, 1).cumsum(2) / torch.arange(1, 201).view(1, 1, 200, 1))
    close(od, want, atol=2e-3, rtol=2e-3)            # Q = 0: running mean of V
    ops.attention(q.cuda(), k.cuda(), v.cuda(), od, 0.1, True)
    torch.cuda.synchronize()
    assert torch.equal(od[:, :, 0].cpu(), v.repeat_interleave(2, 1)[:, :, 0])   # row 0 sees only key 0


def test_attention_token_major_views():
    """q/o as views of token-major [B,S,H*D] buffers (the PreNorm block's layout)."""
    from triton_amd import ops
    B, Hq, Hkv, S, D = 1, 4, 2, 192, 128
    q, k, v = make(B, Hq, Hkv, S, S, D, seed=3)
    qt = q.permute(0, 2, 1, 3).contiguous().cuda()       # [B,S,H,D]
    kt = k.permute(0, 2, 1, 3).contiguous().cuda(); vt = v.permute(0, 2, 1, 3).contiguous().cuda()
    ot = torch.zeros_like(qt)
    ops.attention(qt.permute(0, 2, 1, 3), kt.permute(0, 2, 1, 3), vt.permute(0, 2, 1, 3), ot.permute(0, 2, 1, 3),
                  D ** -0.5, True)
    torch.cuda.synchronize()
    close(ot.permute(0, 2, 1, 3), ref.attention(q, k, v, D ** -0.5, True))


def test_qnorm_fused():
    from triton_amd import ops
    B, Hq, Hkv, S, D = 1, 5, 1, 160, 64
    q, k, v = make(B, Hq, Hkv, S, S, D, seed=11)
    g = torch.Generator().manual_seed(5)
    gq = ref.randn_half((D,), g, 1.0, 0.02); gk = ref.randn_half((D,), g, 1.0, 0.02)
    kd = k.cuda(); kn = torch.empty_like(kd)
    ops.head_rmsnorm(kd.view(B * Hkv, S, D), gk.cuda(), kn.view(B * Hkv, S, D), 1e-5)
    od = torch.zeros_like(q).cuda()
    ops.attention(q.cuda(), kn, v.cuda(), od, D ** -0.5, True, q_norm=True, gamma_q=gq.cuda(), q_eps=1e-5)
    torch.cuda.synchronize()
    close(od, ref.qknorm_attention(q, k, v, gq, gk, 1e-5, D ** -0.5, True))


def test_qnorm_fused_head_dim_128_no_gamma():
    """The query norm of the 16x16x32 kernel sums a row over four lanes; without a weight and with eps = 0 it is the
    reference's QKNorm statement (q * rsqrt(mean(q^2)))."""
    from triton_amd import ops
    B, Hq, Hkv, S, D = 2, 4, 2, 300, 128
    q, k, v = make(B, Hq, Hkv, S, S, D, seed=21)
    od = torch.zeros_like(q).cuda()
    ops.attention(q.cuda(), k.cuda(), v.cuda(), od, D ** -0.5, True, q_norm=True, gamma_q=None, q_eps=0.0)
    torch.cuda.synchronize()
    qn = ref.rmsnorm(q, torch.ones(D, dtype=torch.float16), 0.0)
    close(od, ref.attention(qn, k, v, D ** -0.5, True))


def test_noise_row_normaliser():
    from triton_amd import ops
    B, Hq, Hkv, S, D = 1, 4, 2, 200, 128
    q, k, v = make(B, Hq, Hkv, S, S, D, seed=13)
    noise = ref.gumbel_noise((B, Hq, S, S), 1234)
    od = torch.zeros_like(q).cuda()
    lse = torch.zeros(B, Hq, S, device="cuda"); lsep = torch.zeros(B, Hq, S, device="cuda")
    tau, scale = 1.5, D ** -0.5
    ops.attention(q.cuda(), k.cuda(), v.cuda(), od, scale, True, lse=lse, noise=noise.cuda(), tau=tau, lse_pert=lsep)
    torch.cuda.synchronize()
    close(od, ref.attention(q, k, v, scale, True))
    s = ref.scores_fp32(q, k, scale, True)
    close(lsep, torch.logsumexp((s + noise) / tau, -1), atol=1e-3, rtol=1e-3)
    close(lse, torch.logsumexp(s, -1), atol=1e-3, rtol=1e-3)


def test_attention_bad_arguments():
    from triton_amd import ops, _lib
    q, k, v = make(1, 2, 2, 8, 8, 32)
    with pytest.raises(_lib.TrnError) as e:
        ops.attention(q.cuda(), k.cuda(), v.cuda(), torch.zeros_like(q).cuda(), 1.0, False)
    assert e.value.status_name == "TRN_E_UNSUPPORTED"
    q, k, v = make(1, 3, 2, 8, 8, 64)
    with pytest.raises(_lib.TrnError):
        ops.attention(q.cuda(), k.cuda(), v.cuda(), torch.zeros_like(q).cuda(), 1.0, False)
    q, k, v = make(1, 2, 2, 8, 4, 64)
    with pytest.raises(_lib.TrnError):
        ops.attention(q.cuda(), k.cuda(), v.cuda(), torch.zeros_like(q).cuda(), 1.0, True)   # causal, Skv < Sq
