"""Seeded sweeps over shapes, layouts and element types for the key-score operators and the decode-append modules,
each case held to the CPU oracle.  The fixed cases elsewhere pin the tile edges; these walk the combinations between
them (cached prefixes of any length, 1 to 32 new tokens, fp16 or fp32 noise and score tensors, both output
placements), the way the reference's drivers would call the modules (convert_eval_rms.py:146-160, 201)."""
import random

import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def off(got, want, rtol, atol):
    got = got.float().cpu(); want = want.float()
    err = (got - want).abs()
    return int((err > atol + rtol * want.abs()).sum()), float(err.max())


def _score_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        kind = rnd.choice(("roco", "keyformer", "fused"))
        D = rnd.choice((64, 128)); Hkv = rnd.choice((1, 2, 3)); Hq = Hkv * rnd.choice((1, 2, 4)); B = rnd.choice((1, 1, 2))
        causal = rnd.random() < 0.6
        if kind == "fused":
            Sq = rnd.choice((1, 7, 16, 32)); Skv = Sq + rnd.choice((0, 100, 333, 1024, 2500))
        else:
            Sq = rnd.choice((1, 33, 64, 100, 129, 255, 300, 512, 640, 777, 1100))
            Skv = Sq + rnd.choice((0, 0, 1, 31, 64, 257, 1000)) if causal else rnd.choice((1, 17, 64, 65, 200, 333, 512, 700, 1100))
            if kind == "keyformer":
                Sq, Skv = min(Sq, 640), min(Skv, 900) if not causal else min(Sq, 640) + min(Skv - Sq, 257)
        out.append((kind, B, Hq, Hkv, Sq, Skv, D, causal, rnd.randrange(1 << 20)))
    return out


@pytest.mark.parametrize("kind,B,Hq,Hkv,Sq,Skv,D,causal,seed", _score_cases(40, 20260214))
def test_key_score_operators_seeded_shapes(kind, B, Hq, Hkv, Sq, Skv, D, causal, seed):
    from triton_amd import ops
    g = torch.Generator().manual_seed(seed)
    q, k, v = ref.randn_half((B, Hq, Sq, D), g), ref.randn_half((B, Hkv, Skv, D), g), ref.randn_half((B, Hkv, Skv, D), g)
    scale = D ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros_like(qd); lse = torch.zeros(B, Hq, Sq, device="cuda")
    s1 = torch.full((B, Hq, Skv), -1.0, device="cuda"); s2 = torch.full((B, Hq, Skv), -1.0, device="cuda")
    if kind == "keyformer":
        tau = 1.5
        noise = ref.gumbel_noise((B, Hq, Sq, Skv), seed)
        pitch = (Skv + 3) // 4 * 4          # the kernels fetch noise 16 bytes at a time: padded rows, NaN in the padding
        nd = torch.full((B, Hq, Sq, pitch), float("nan")); nd[..., :Skv] = noise; nd = nd.cuda()[..., :Skv]
        ops.attention(qd, kd, vd, o, scale, causal, noise=nd, tau=tau, lse_pert=lse)
        ops.attention_colstats(qd, kd, lse, scale, causal, s1, None, noise=nd, tau=tau)
        wo, w1 = ref.keyformer(q, k, v, noise, scale, tau, causal)
        res = [off(o, wo, 1e-2, 2e-2), off(s1, w1, 1e-3, 1e-5)]
    else:
        if kind == "fused":
            ops.attention_with_stats(qd, kd, vd, o, scale, causal, s1, s2, lse=lse)
        else:
            ops.attention(qd, kd, vd, o, scale, causal, lse=lse)
            ops.attention_colstats(qd, kd, lse, scale, causal, s1, s2)
        wo, w1, w2 = ref.roco(q, k, v, scale, causal)
        # (a sum of squares carries twice the relative error of the probabilities under it)
        res = [off(o, wo, 1e-2, 2e-2), off(s1, w1, 1e-3, 1e-5), off(s2, w2, 2e-3, 1e-5)]
    torch.cuda.synchronize()
    assert not any(c for c, _ in res), res


def _module_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        v = rnd.choice(("vanilla", "prenorm", "qknorm", "keyformer", "keyformer", "roco", "roco"))
        D = rnd.choice((64, 128)); H = rnd.choice((1, 2, 3, 5, 8))
        M = rnd.choice((1, 3, 8, 16, 17, 32)); P = rnd.choice((0, 1, 31, 100, 257, 1024, 1500, 3000))
        out.append((v, H, D, M, P, rnd.choice(("token_major", "head_major")), rnd.choice(("f16", "f32")),
                    rnd.choice(("f16", "f32")), rnd.randrange(1 << 20)))
    return out


@pytest.mark.parametrize("variant,H,D,M,P,layout,score_dt,noise_dt,seed", _module_cases(60, 20260215))
def test_decode_append_modules_seeded_shapes_layouts_and_dtypes(variant, H, D, M, P, layout, score_dt, noise_dt, seed):
    from triton_amd import modules
    dt = {"f16": torch.float16, "f32": torch.float32}
    g = torch.Generator().manual_seed(seed)
    N = H * D
    r = lambda *s: (torch.randn(*s, generator=g).clamp(-1, 1) * 0.05).half()
    # (WQ, WK small: the reference's classes use no 1/sqrt(D) scale, and PreNorm's unit-RMS rows would otherwise give
    # scores in the hundreds, where any two fp16 roundings of Q and K disagree on the softmax)
    X, WQ, WK, WV = r(M, N), r(N, N) * 0.2, r(N, N) * 0.2, r(N, N)
    Kc, Vc = r(H, P + M, D) * 4, r(H, P + M, D) * 4
    t = dict(X=X.cuda(), WQ=WQ.cuda(), WK=WK.cuda(), WV=WV.cuda(), K_cache=Kc.cuda(), V_cache=Vc.cuda(),
             O2=torch.zeros(M, N, dtype=torch.float16, device="cuda"))
    flat = ref.flatten_token_major if layout == "token_major" else ref.flatten_head_major
    want = []
    if variant in ("vanilla", "prenorm"):
        wo = ref.decode_append_vanilla(X, WQ, WK, WV, Kc, Vc, P, D, variant == "prenorm")
    elif variant == "qknorm":
        wo = ref.decode_append_qknorm(X, WQ, WK, WV, Kc, Vc, P, D)
    elif variant == "keyformer":
        noise = torch.randn(H, M, P + M, generator=g).to(dt[noise_dt])
        t["noise"] = noise.cuda(); t["C_out"] = torch.zeros(H, P + M, dtype=dt[score_dt], device="cuda")
        wo, pw = ref.decode_append_keyformer(X, WQ, WK, WV, Kc, Vc, noise.float(), P, D, 1.5)
        want = [("C_out", pw.sum(1))]
    else:
        t["C_out1"] = torch.zeros(H, P + M, dtype=dt[score_dt], device="cuda"); t["C_out2"] = torch.zeros_like(t["C_out1"])
        wo, w1, w2 = ref.decode_append_roco(X, WQ, WK, WV, Kc, Vc, P, D)
        want = [("C_out1", w1), ("C_out2", w2)]
    m = modules.get(variant, "decode", head_dim=D, o_layout=layout)
    m.forward(*[t[p] for p in m.TENSOR_PARAMS])
    torch.cuda.synchronize()
    half = score_dt == "f16"         # an fp16 score tensor adds its own rounding
    res = [off(t["O2"], flat(wo), 1e-2, 2e-2)] + [off(t[k_], w_, 2e-3 if half else 1e-3, 1e-3 if half else 1e-5) for k_, w_ in want]
    assert not any(c for c, _ in res), res
