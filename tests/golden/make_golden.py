"""Writes tests/golden/kat_small.npz: small known-answer vectors for the six operators, LoRA and the gated MLP.

The reference ships no golden vectors for this path, so these come from the fp64 loop-level definitions in
oracle/brute.py (written from the mathematics, independently of oracle/ref.py's tensor expressions) on seeded fp16
inputs.  They freeze today's agreed answers: oracle/ref.py and the HIP kernels are both checked against the file, so
a later change to either shows up against a third, fixed party.

    python tests/golden/make_golden.py          # regenerates the file (deterministic)
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import brute  # noqa: E402


def h16(rng, shape, std=1.0, mean=0.0):
    return (mean + std * rng.standard_normal(shape)).astype(np.float16)


def head_norm(t, gamma, eps):
    """Per-head RMSNorm over the last axis, rounded to fp16 as the normalised q/k tensors are (ref_rms.py:217-222)."""
    out = np.stack([brute.rmsnorm(t[h].astype(np.float64), gamma.astype(np.float64), eps) for h in range(t.shape[0])])
    return out.astype(np.float16)


def main():
    rng = np.random.default_rng(20240611)
    out = {}
    # RMSNorm with gamma and eps (ref_attn.py:348-350) and bare (ref_rms.py:102-103)
    x = h16(rng, (6, 64)); g = h16(rng, (64,), 0.02, 1.0)
    out.update(rms_x=x, rms_gamma=g, rms_eps=np.float32(1e-5), rms_y=brute.rmsnorm(x, g.astype(np.float64), 1e-5),
               rms_y_bare=brute.rmsnorm(x, None, 0.0))
    # causal GQA attention with column statistics and KeyFormer scores
    q = h16(rng, (4, 12, 64)); k = h16(rng, (2, 12, 64)); v = h16(rng, (2, 12, 64))
    u = np.clip(rng.random((4, 12, 12)), 1e-10, 1 - 1e-7)
    noise = (-np.log(-np.log(u))).astype(np.float32)
    r = brute.attention_all(q, k, v, 0.125, True, noise, 1.5)
    out.update(gqa_q=q, gqa_k=k, gqa_v=v, gqa_scale=np.float32(0.125), gqa_noise=noise, gqa_tau=np.float32(1.5),
               gqa_o=r["o"], gqa_lse=r["lse"], gqa_colsum=r["colsum"], gqa_colsumsq=r["colsumsq"],
               gqa_pert_colsum=r["pert_colsum"])
    # the reference's own semantics: no scale, no mask, a cached prefix (5 new tokens, 13 keys), MHA
    q = h16(rng, (2, 5, 64), 0.3); k = h16(rng, (2, 13, 64), 0.3); v = h16(rng, (2, 13, 64))
    r = brute.attention_all(q, k, v, 1.0, False)
    out.update(pre_q=q, pre_k=k, pre_v=v, pre_o=r["o"], pre_lse=r["lse"], pre_colsum=r["colsum"], pre_colsumsq=r["colsumsq"])
    # QK-norm MQA
    q = h16(rng, (3, 9, 64)); k = h16(rng, (1, 9, 64)); v = h16(rng, (1, 9, 64))
    gq = h16(rng, (64,), 0.02, 1.0); gk = h16(rng, (64,), 0.02, 1.0)
    r = brute.attention_all(head_norm(q, gq, 1e-5), head_norm(k, gk, 1e-5), v, 0.125, True)
    out.update(qkn_q=q, qkn_k=k, qkn_v=v, qkn_gq=gq, qkn_gk=gk, qkn_eps=np.float32(1e-5), qkn_o=r["o"])
    # RMSNorm fused into the Q/K/V projections (X @ W, ref_rms.py:102-107)
    x = h16(rng, (7, 64)); g = h16(rng, (64,), 0.02, 1.0)
    wq = h16(rng, (64, 128), 0.05); wk = h16(rng, (64, 64), 0.05); wv = h16(rng, (64, 64), 0.05)
    xn = brute.rmsnorm(x, g.astype(np.float64), 1e-5)
    out.update(prj_x=x, prj_gamma=g, prj_wq=wq, prj_wk=wk, prj_wv=wv, prj_eps=np.float32(1e-5),
               prj_q=xn @ wq.astype(np.float64), prj_k=xn @ wk.astype(np.float64), prj_v=xn @ wv.astype(np.float64))
    # LoRA (lora_benchmark.py:41-53) and the two gates of the gated MLP (gmlp_benchmark.py:53-64), in fp64 from the
    # definitions (drawn last, so that the vectors above stay as they were)
    x = h16(rng, (5, 64), 0.5); w = h16(rng, (64, 48), 0.05); la = h16(rng, (64, 8), 0.05); lb = h16(rng, (8, 48), 0.2)
    x64 = x.astype(np.float64)
    out.update(lora_x=x, lora_w=w, lora_a=la, lora_b=lb,
               lora_o=x64 @ w.astype(np.float64) + (x64 @ la.astype(np.float64)) @ lb.astype(np.float64))
    w1 = h16(rng, (64, 40), 0.1); w2 = h16(rng, (64, 40), 0.1)
    c1 = x64 @ w1.astype(np.float64); c2 = x64 @ w2.astype(np.float64)
    sg = 1.0 / (1.0 + np.exp(-c1))
    out.update(gmlp_x=x, gmlp_w1=w1, gmlp_w2=w2, gmlp_o_sigmoid=sg * c2, gmlp_o_silu=c1 * sg * c2)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_small.npz")
    np.savez_compressed(path, **{n: (a if a.dtype in (np.float16, np.float32) else np.asarray(a, np.float32))
                                 for n, a in ((n, np.asarray(a)) for n, a in out.items())})
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
