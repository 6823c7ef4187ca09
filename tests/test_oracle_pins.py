"""Pins for oracle/ref.py: closed forms, invariants, library routines and fp64 brute
force.  The reference holds no tests or golden vectors for this path, so these are
what fixes the oracle; each targets a plausible mistake (dropped eps, wrong GQA head
map, off-by-one diagonal, transposed operand, wrong tau placement...)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute, ref


def gen(seed=0):
    return torch.Generator(device="cpu").manual_seed(seed)


# ------------------------------------------------------------------ RMSNorm
def test_rmsnorm_constant_row_is_sign():
    x = torch.full((3, 16), -2.5).half()
    assert torch.equal(ref.rmsnorm(x), torch.full((3, 16), -1.0).half())


def test_rmsnorm_matches_library_routine():
    g = gen(1)
    x = ref.randn_half((37, 256), g)
    w = ref.randn_half((256,), g, 1.0, 0.02)
    lib = F.rms_norm(x.float(), (256,), w.float(), 1e-5).half()
    assert torch.equal(ref.rmsnorm(x, w, 1e-5), lib)


def test_rmsnorm_mean_square_identity_and_scale_equivariance():
    g = gen(2)
    x = torch.randn(5, 64, generator=g)
    eps = 0.3
    y = ref.rmsnorm(x, None, eps)
    ms = x.pow(2).mean(-1)
    assert torch.allclose(y.pow(2).mean(-1), ms / (ms + eps), rtol=1e-5)
    assert torch.allclose(ref.rmsnorm(7.0 * x), ref.rmsnorm(x), rtol=1e-5, atol=1e-6)


def test_rmsnorm_brute_fp64():
    g = gen(3)
    x = torch.randn(4, 8, generator=g); w = torch.randn(8, generator=g)
    got = ref.rmsnorm(x, w, 1e-5).double().numpy()
    np.testing.assert_allclose(got, brute.rmsnorm(x.numpy(), w.numpy(), 1e-5), rtol=2e-6)


# ------------------------------------------------------------------ attention
def _qkv(g, B, Hq, Hkv, Sq, Skv, D, dtype=torch.float32):
    q = torch.randn(B, Hq, Sq, D, generator=g).to(dtype)
    k = torch.randn(B, Hkv, Skv, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, Skv, D, generator=g).to(dtype)
    return q, k, v


@pytest.mark.parametrize("causal", [False, True])
def test_attention_matches_sdpa(causal):
    g = gen(4)
    q, k, v = _qkv(g, 2, 8, 2, 33, 33, 16)
    scale = 16 ** -0.5
    lib = F.scaled_dot_product_attention(q, k.repeat_interleave(4, 1), v.repeat_interleave(4, 1),
                                         is_causal=causal, scale=scale)
    assert torch.allclose(ref.attention(q, k, v, scale, causal), lib, rtol=1e-5, atol=1e-6)


def test_attention_causal_row0_and_uniform():
    g = gen(5)
    q, k, v = _qkv(g, 1, 4, 2, 9, 9, 8)
    o = ref.attention(q, k, v, 0.3, True)
    assert torch.allclose(o[:, :, 0], v.repeat_interleave(2, 1)[:, :, 0], atol=1e-6)
    o0 = ref.attention(torch.zeros_like(q), k, v, 0.3, True)
    want = v.repeat_interleave(2, 1).cumsum(2) / torch.arange(1, 10).view(1, 1, 9, 1)
    assert torch.allclose(o0, want, atol=1e-6)


def test_attention_prefix_causal_sees_prefix():
    # Sq < Skv: query i sees keys <= (Skv-Sq)+i.
    g = gen(6)
    q, k, v = _qkv(g, 1, 2, 2, 3, 7, 4)
    o = ref.attention(torch.zeros_like(q), k, v, 1.0, True)
    for i in range(3):
        assert torch.allclose(o[0, :, i], v[0, :, : 5 + i].mean(1), atol=1e-6)


def test_attention_gqa_equals_mha_with_replicated_kv_and_head_permutation():
    g = gen(7)
    q, k, v = _qkv(g, 1, 6, 3, 5, 5, 4)
    a = ref.attention(q, k, v, 0.5, True)
    b = ref.attention(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), 0.5, True)
    assert torch.equal(a, b)
    perm = torch.tensor([5, 3, 1, 0, 2, 4])
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    c = ref.attention(q[:, perm], kk[:, perm], vv[:, perm], 0.5, True)
    assert torch.equal(c, b[:, perm])


@pytest.mark.parametrize("causal", [False, True])
def test_attention_brute_fp64(causal):
    g = gen(8)
    q, k, v = _qkv(g, 1, 4, 2, 5, 7, 4)
    noise = torch.randn(4, 5, 7, generator=g)
    bf = brute.attention_all(q[0].numpy(), k[0].numpy(), v[0].numpy(), 0.7, causal, noise.numpy(), 1.5)
    o, lse = ref.attention(q, k, v, 0.7, causal, return_lse=True)
    np.testing.assert_allclose(o[0].double().numpy(), bf["o"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(lse[0].double().numpy(), bf["lse"], rtol=1e-5, atol=1e-6)
    _, s1, s2 = ref.roco(q, k, v, 0.7, causal)
    np.testing.assert_allclose(s1[0].double().numpy(), bf["colsum"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(s2[0].double().numpy(), bf["colsumsq"], rtol=1e-5, atol=1e-6)
    _, kf = ref.keyformer(q, k, v, noise[None], 0.7, 1.5, causal)
    np.testing.assert_allclose(kf[0].double().numpy(), bf["pert_colsum"], rtol=1e-5, atol=1e-6)
    _, pw = ref.keyformer(q, k, v, noise[None], 0.7, 1.5, causal, reduce=False)
    np.testing.assert_allclose(pw[0].double().numpy(), bf["pert"], rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ QKNorm
def test_qknorm_scale_invariance_and_bound():
    g = gen(9)
    q, k, v = _qkv(g, 1, 3, 1, 6, 6, 8)
    a = ref.qknorm_attention(q, k, v, None, None, 0.0, 0.4, True)
    qs = q * torch.rand(1, 3, 6, 1, generator=g).add(0.5)
    ks = k * torch.rand(1, 1, 6, 1, generator=g).add(0.5)
    assert torch.allclose(ref.qknorm_attention(qs, ks, v, None, None, 0.0, 0.4, True), a, atol=1e-5)
    qn, kn = ref.head_rmsnorm(q, None, 0.0), ref.head_rmsnorm(k, None, 0.0)
    assert torch.allclose(qn.pow(2).mean(-1), torch.ones(1, 3, 6), atol=1e-5)
    assert (qn @ kn.transpose(-1, -2)).abs().max() <= 8 + 1e-4
    assert torch.allclose(ref.attention(qn, kn, v, 0.4, True), a, atol=1e-6)


def test_qknorm_prefix_not_renormed():
    g = gen(10)
    q, k, v = _qkv(g, 1, 2, 2, 2, 5, 4)
    kn = ref.head_rmsnorm(k, None, 0.0, start=3)
    assert torch.equal(kn[..., :3, :], k[..., :3, :])
    assert torch.allclose(kn[..., 3:, :].pow(2).mean(-1), torch.ones(1, 2, 2), atol=1e-5)


# ------------------------------------------------------------------ key scores
def test_keyformer_rows_sum_to_queries_and_zero_noise_equals_roco():
    g = gen(11)
    q, k, v = _qkv(g, 1, 4, 2, 6, 6, 8)
    noise = ref.gumbel_noise((1, 4, 6, 6), 3)
    _, kf = ref.keyformer(q, k, v, noise, 0.35, 1.0, True)
    assert torch.allclose(kf.sum(-1), torch.full((1, 4), 6.0), atol=1e-5)
    _, kf0 = ref.keyformer(q, k, v, torch.zeros_like(noise), 0.35, 1.0, True)
    _, s1, s2 = ref.roco(q, k, v, 0.35, True)
    assert torch.allclose(kf0, s1, atol=1e-6)
    assert (s2 >= 0).all() and (s2 <= s1 + 1e-6).all()
    assert torch.allclose(s1.sum(-1), torch.full((1, 4), 6.0), atol=1e-5)


def test_uniform_attention_harmonic_closed_forms():
    S = 40
    g = gen(12)
    q, k, v = _qkv(g, 1, 2, 1, S, S, 4)
    q = torch.zeros_like(q)
    _, s1, s2 = ref.roco(q, k, v, 1.0, True)
    assert torch.allclose(s1[0, 0].double(), ref.harmonic_tail(S, 1), rtol=1e-5)
    assert torch.allclose(s2[0, 1].double(), ref.harmonic_tail(S, 2), rtol=1e-5)
    _, kf = ref.keyformer(q, k, v, torch.zeros(1, 2, S, S), 1.0, 1.0, True)
    assert torch.allclose(kf[0, 0].double(), ref.harmonic_tail(S, 1), rtol=1e-5)
    mean, std = ref.roco_mean_std(s1, s2, S, True)
    # under uniform attention key j's visible probabilities are 1/(i+1), i>=j
    j = 7
    pj = 1.0 / torch.arange(j + 1, S + 1, dtype=torch.float64)
    assert math.isclose(mean[0, 0, j].item(), pj.mean().item(), rel_tol=1e-5)
    assert math.isclose(std[0, 0, j].item(), pj.std(unbiased=False).item(), rel_tol=1e-4)


def test_roco_mean_std_is_numpy_mean_and_std_over_the_visible_rows():
    """The convention of roco_mean_std, stated by what it must equal: numpy's mean and (population) std of column j of
    the probability matrix, taken over the rows that can see key j."""
    g = gen(21)
    Sq, Skv = 9, 14
    q, k, v = _qkv(g, 1, 2, 1, Sq, Skv, 8)
    for causal in (True, False):
        _, s1, s2 = ref.roco(q, k, v, 0.7, causal)
        mean, std = ref.roco_mean_std(s1, s2, Sq, causal)
        p = torch.softmax(ref.scores_fp32(q, k, 0.7, causal).double(), -1).numpy()
        for j in range(Skv):
            first = max(0, j - (Skv - Sq)) if causal else 0
            col = p[0, :, first:, j]
            assert np.allclose(mean[0, :, j].numpy(), col.mean(-1), rtol=1e-5)
            assert np.allclose(std[0, :, j].numpy(), col.std(-1), rtol=1e-3, atol=1e-6)


def test_tau_divides_both_score_and_noise():
    # (s + g)/tau, not s/tau + g and not s + g/tau: with tau=2 and doubled s, g it is the tau=1 result.
    g = gen(13)
    q, k, v = _qkv(g, 1, 2, 2, 4, 4, 4)
    noise = torch.randn(1, 2, 4, 4, generator=g)
    _, a = ref.keyformer(q, k, v, noise, 1.0, 1.0, False)
    _, b = ref.keyformer(2 * q, k, v, 2 * noise, 1.0, 2.0, False)
    assert torch.allclose(a, b, atol=1e-6)


def test_gumbel_generator_definition():
    a = ref.gumbel_noise((4, 5), 99); b = ref.gumbel_noise((4, 5), 99)
    assert torch.equal(a, b)
    u = torch.rand((4, 5), generator=gen(99)).clamp_(1e-10, 1 - 1e-7)
    assert torch.equal(a, -torch.log(-torch.log(u)))
    big = ref.gumbel_noise((200000,), 5)
    assert abs(big.mean().item() - 0.5772) < 0.02 and abs(big.var().item() - math.pi ** 2 / 6) < 0.05


# ------------------------------------------------------------------ PreNorm + decode-append forms
def test_prenorm_block_composition_and_row_scale_identity():
    g = gen(14)
    B, S, N, D, Hkv = 1, 6, 32, 8, 2
    x = ref.randn_half((B, S, N), g)
    gamma = ref.randn_half((N,), g, 1.0, 0.02)
    wq = ref.randn_half((N, N), g, 0, 0.1); wk = ref.randn_half((N, Hkv * D), g, 0, 0.1); wv = ref.randn_half((N, Hkv * D), g, 0, 0.1)
    o = ref.prenorm_block(x, gamma, wq, wk, wv, D, 1e-5, D ** -0.5, True)
    assert o.shape == (B, S, N)
    # per-head column slicing witnessed by the loop form (convert_eval_rms.py:132-160)
    xn = ref.rmsnorm(x, gamma, 1e-5).float()[0]
    for h in range(N // D):
        hk = h // ((N // D) // Hkv)
        qh = (xn @ wq.float()[:, h * D:(h + 1) * D]).half()
        kh = (xn @ wk.float()[:, hk * D:(hk + 1) * D]).half()
        vh = (xn @ wv.float()[:, hk * D:(hk + 1) * D]).half()
        oh = ref.attention(qh[None, None], kh[None, None], vh[None, None], D ** -0.5, True)[0, 0]
        assert torch.equal(o[0, :, h * D:(h + 1) * D], oh)
    # (x * r) @ W == r * (x @ W) in exact arithmetic
    xf = x.float()[0]; r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)
    assert torch.allclose((xf * r * gamma.float()) @ wq.float(), r * ((xf * gamma.float()) @ wq.float()), rtol=1e-4, atol=1e-5)


def _decode_inputs(g, M=4, N=32, D=8, P=5):
    H = N // D
    X = ref.reference_recipe((M, N), g) * 50
    W = [ref.reference_recipe((N, N), g) * 50 for _ in range(3)]
    Kc = ref.reference_recipe((H, P + M, D), g) * 50
    Vc = ref.reference_recipe((H, P + M, D), g) * 50
    return X, W, Kc, Vc, M, N, D, P, H


def test_decode_append_vanilla_line_by_line():
    g = gen(15)
    X, W, Kc, Vc, M, N, D, P, H = _decode_inputs(g)
    o = ref.decode_append_vanilla(X, *W, Kc, Vc, P, D)
    # independent restatement in fp32 of ref_rms.py:47-81
    q = (X.float() @ W[0].float()).half().view(M, H, D)
    k = (X.float() @ W[1].float()).half().view(M, H, D).transpose(0, 1)
    v = (X.float() @ W[2].float()).half().view(M, H, D).transpose(0, 1)
    kc = torch.cat([Kc[:, :P], k], 1).float(); vc = torch.cat([Vc[:, :P], v], 1).float()
    w = F.softmax(q.transpose(0, 1).float() @ kc.transpose(1, 2), dim=-1)
    want = (w @ vc).half()
    assert torch.equal(o, want)
    assert ref.flatten_head_major(o).shape == (M, N)
    tm = ref.flatten_token_major(o)
    assert torch.equal(tm[:, D:2 * D], o[1])


def test_decode_append_qknorm_brute_force_and_what_is_normalised():
    """QKNorm.forward (ref_rms.py:205-229): q and the NEW k rows are divided by their root mean square over head_dim
    (no eps, no weight), the cached prefix is used as stored, scores unscaled and unmasked.  Pinned by an fp64
    loop-level definition, and by what the normalisation implies: the result does not change when W_q or W_k is
    scaled, but does change when the cached prefix of K is (normalising the whole cache would hide that)."""
    g = gen(17)
    X, W, Kc, Vc, M, N, D, P, H = _decode_inputs(g)
    o = ref.decode_append_qknorm(X, *W, Kc, Vc, P, D)
    Xd = X.double().numpy(); Wd = [w.double().numpy() for w in W]
    want = np.zeros((H, M, D))
    for h in range(H):
        # fp16-rounded projections, as the reference's half-precision matmul leaves them
        q = np.array([[np.float16(sum(Xd[m, n] * Wd[0][n, h * D + d] for n in range(N))) for d in range(D)] for m in range(M)], dtype=np.float64)
        k = np.array([[np.float16(sum(Xd[m, n] * Wd[1][n, h * D + d] for n in range(N))) for d in range(D)] for m in range(M)], dtype=np.float64)
        v = np.array([[np.float16(sum(Xd[m, n] * Wd[2][n, h * D + d] for n in range(N))) for d in range(D)] for m in range(M)], dtype=np.float64)
        for m in range(M):
            qn = np.float16(q[m] / math.sqrt(sum(x * x for x in q[m]) / D)).astype(np.float64)
            keys = [Kc[h, j].double().numpy() for j in range(P)]
            vals = [Vc[h, j].double().numpy() for j in range(P)]
            for j in range(M):
                keys.append(np.float16(k[j] / math.sqrt(sum(x * x for x in k[j]) / D)).astype(np.float64))
                vals.append(v[j])
            s = [sum(qn[d] * kj[d] for d in range(D)) for kj in keys]
            mx = max(s)
            e = [math.exp(x - mx) for x in s]
            z = sum(e)
            for d in range(D):
                want[h, m, d] = sum(e[j] * vals[j][d] for j in range(P + M)) / z
    assert np.abs(o.double().numpy() - want).max() < 2e-3 * max(1.0, np.abs(want).max())
    # invariant under the scale of W_q and of W_k (powers of two: exact in fp16) ...
    o_q = ref.decode_append_qknorm(X, W[0] * 4, W[1], W[2], Kc, Vc, P, D)
    o_k = ref.decode_append_qknorm(X, W[0], W[1] * 0.5, W[2], Kc, Vc, P, D)
    assert torch.allclose(o_q.float(), o.float(), atol=2e-3) and torch.allclose(o_k.float(), o.float(), atol=2e-3)
    # ... but not under the scale of the cached prefix, which is not normalised
    Kc2 = Kc.clone(); Kc2[:, :P] *= 8
    o_c = ref.decode_append_qknorm(X, *W, Kc2, Vc, P, D)
    assert (o_c.float() - o.float()).abs().max() > 1e-2
    # and the rows P.. of the cache that come in are ignored (they are overwritten by the new keys)
    Kc3 = Kc.clone(); Kc3[:, P:] = 9.0
    assert torch.equal(ref.decode_append_qknorm(X, *W, Kc3, Vc, P, D), o)


def test_decode_append_variants_consistent():
    g = gen(16)
    X, W, Kc, Vc, M, N, D, P, H = _decode_inputs(g)
    o = ref.decode_append_vanilla(X, *W, Kc, Vc, P, D)
    noise = torch.randn(H, M, P + M, generator=g).half()
    ok, pw = ref.decode_append_keyformer(X, *W, Kc, Vc, noise, P, D)
    assert torch.equal(ok, o) and pw.shape == (H, M, P + M)
    assert torch.allclose(pw.sum(-1), torch.ones(H, M), atol=1e-5)
    orc, s1, s2 = ref.decode_append_roco(X, *W, Kc, Vc, P, D)
    assert torch.equal(orc, o) and torch.allclose(s1.sum(-1), torch.full((H,), float(M)), atol=1e-4)
    op = ref.decode_append_vanilla(X, *W, Kc, Vc, P, D, prenorm=True)
    o2 = ref.decode_append_vanilla(ref.rmsnorm(X), *W, Kc, Vc, P, D)
    assert torch.equal(op, o2)
    oq = ref.decode_append_qknorm(X, *W, Kc, Vc, P, D)
    assert oq.shape == (H, M, D) and torch.isfinite(oq.float()).all()


def test_lora_closed_forms_and_brute_force():
    """O = X W + (X A) B: zero adapter, zero base, rank-1 adapter in closed form, fp64 brute force."""
    g = torch.Generator().manual_seed(7)
    M, N, P, R = 5, 24, 16, 8
    X, W = ref.randn_half((M, N), g, 0, 0.5), ref.randn_half((N, P), g, 0, 0.5)
    A, B = ref.randn_half((N, R), g, 0, 0.5), ref.randn_half((R, P), g, 0, 0.5)
    zA, zW = torch.zeros_like(A), torch.zeros_like(W)
    assert torch.equal(ref.lora(X, W, zA, B), (X.float() @ W.float()).half())                 # adapter off
    assert torch.equal(ref.lora(X, zW, A, B), ((X.float() @ A.float()).half().float() @ B.float()).half())
    # rank 1: (X a) b^T adds (x_i . a) * b_j
    a1 = torch.zeros_like(A); a1[:, 0] = A[:, 0]
    b1 = torch.zeros_like(B); b1[0] = B[0]
    want = X.double() @ W.double() + torch.outer(X.double() @ a1[:, 0].double(), b1[0].double())
    assert torch.allclose(ref.lora(X, W, a1, b1).double(), want, rtol=2e-3, atol=2e-3)
    brute = torch.zeros(M, P, dtype=torch.float64)
    for i in range(M):
        for j in range(P):
            acc = sum(float(X[i, k]) * float(W[k, j]) for k in range(N))
            acc += sum(sum(float(X[i, k]) * float(A[k, r]) for k in range(N)) * float(B[r, j]) for r in range(R))
            brute[i, j] = acc
    assert torch.allclose(ref.lora(X, W, A, B).double(), brute, rtol=4e-3, atol=4e-3)
    # the identity the fused form rests on: X W + (X A) B = X (W + A B)
    assert torch.allclose(ref.lora(X, W, A, B).double(), X.double() @ (W.double() + A.double() @ B.double()), rtol=4e-3, atol=4e-3)


def test_gated_mlp_parts_and_special_values():
    """gate(X W1) * (X W2): W1 = 0 gives sigmoid(0) = 1/2 (sigmoid gate) or 0 (SiLU); library sigmoid / silu."""
    g = torch.Generator().manual_seed(9)
    X, W1, W2 = ref.randn_half((6, 32), g, 0, 0.5), ref.randn_half((32, 16), g, 0, 0.5), ref.randn_half((32, 16), g, 0, 0.5)
    c2 = (X.float() @ W2.float()).half().float()
    assert torch.equal(ref.gated_mlp(X, torch.zeros_like(W1), W2), (0.5 * c2).half())
    assert torch.equal(ref.gated_mlp(X, torch.zeros_like(W1), W2, "silu"), torch.zeros(6, 16, dtype=torch.float16))
    c1 = (X.float() @ W1.float()).half().float()
    assert torch.equal(ref.gated_mlp(X, W1, W2, "silu"), (torch.nn.functional.silu(c1) * c2).half())
    want = (1.0 / (1.0 + torch.exp(-c1.double()))) * c2.double()
    assert torch.allclose(ref.gated_mlp(X, W1, W2).double(), want, rtol=1e-3, atol=1e-3)
    with pytest.raises(ValueError):
        ref.gated_mlp(X, W1, W2, "relu")
