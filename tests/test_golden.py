"""Known-answer vectors (tests/golden/kat_small.npz, fp64 loop-level definitions on seeded fp16 inputs; made by
tests/golden/make_golden.py).  The CPU oracle and the HIP kernels are each held to the same file.
Tolerances: fp16 outputs atol 2e-2 / rtol 1e-2 for the kernels (the fp32 oracle is held to fp16 rounding: 2e-3),
RMSNorm 1e-3 relative, fp32 row normalisers and key scores 1e-3 relative."""
import os

import numpy as np
import pytest
import torch

from oracle import ref

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "kat_small.npz"))


def T(name):
    return torch.from_numpy(G[name])


def close(got, want, atol, rtol):
    got = got.float().cpu(); want = want.float()
    err = (got - want).abs()
    assert (err <= atol + rtol * want.abs()).all(), f"max abs err {err.max():.4g}"


# ------------------------------------------------------------------ the CPU oracle against the vectors
def test_oracle_rmsnorm_kat():
    close(ref.rmsnorm(T("rms_x"), T("rms_gamma"), float(G["rms_eps"])), T("rms_y"), 2e-3, 1e-3)
    close(ref.rmsnorm(T("rms_x"), None, 0.0), T("rms_y_bare"), 2e-3, 1e-3)


def test_oracle_attention_scores_kat():
    q, k, v = T("gqa_q")[None], T("gqa_k")[None], T("gqa_v")[None]
    scale, tau = float(G["gqa_scale"]), float(G["gqa_tau"])
    o, lse = ref.attention(q, k, v, scale, True, return_lse=True)
    close(o[0], T("gqa_o"), 2e-3, 1e-3); close(lse[0], T("gqa_lse"), 1e-5, 1e-5)
    _, s1, s2 = ref.roco(q, k, v, scale, True)
    close(s1[0], T("gqa_colsum"), 1e-6, 1e-4); close(s2[0], T("gqa_colsumsq"), 1e-6, 1e-4)
    _, sc = ref.keyformer(q, k, v, T("gqa_noise")[None], scale, tau, True)
    close(sc[0], T("gqa_pert_colsum"), 1e-6, 1e-4)
    q, k, v = T("pre_q")[None], T("pre_k")[None], T("pre_v")[None]
    o, s1, s2 = ref.roco(q, k, v, 1.0, False)
    close(o[0], T("pre_o"), 2e-3, 1e-3); close(s1[0], T("pre_colsum"), 1e-6, 1e-4); close(s2[0], T("pre_colsumsq"), 1e-6, 1e-4)


def test_oracle_qknorm_and_projection_kat():
    o = ref.qknorm_attention(T("qkn_q")[None], T("qkn_k")[None], T("qkn_v")[None], T("qkn_gq"), T("qkn_gk"),
                             float(G["qkn_eps"]), 0.125, True)
    close(o[0], T("qkn_o"), 2e-3, 1e-3)
    q, k, v = ref.qkv_project(T("prj_x")[None], T("prj_gamma"), T("prj_wq"), T("prj_wk"), T("prj_wv"), float(G["prj_eps"]))
    close(q[0], T("prj_q"), 2e-3, 2e-3); close(k[0], T("prj_k"), 2e-3, 2e-3); close(v[0], T("prj_v"), 2e-3, 2e-3)


# ------------------------------------------------------------------ the HIP kernels against the vectors
@pytest.mark.gpu
def test_hip_rmsnorm_kat():
    from triton_amd import ops
    x = T("rms_x").cuda(); y = torch.empty_like(x)
    ops.rmsnorm(x, T("rms_gamma").cuda(), y, float(G["rms_eps"]))
    close(y, T("rms_y"), 2e-3, 1e-3)
    ops.rmsnorm(x, None, y, 0.0)
    close(y, T("rms_y_bare"), 2e-3, 1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("case,causal", [("gqa", True), ("pre", False)])
def test_hip_attention_scores_kat(case, causal):
    from triton_amd import ops
    q, k, v = T(case + "_q")[None].cuda(), T(case + "_k")[None].cuda(), T(case + "_v")[None].cuda()
    scale = float(G["gqa_scale"]) if case == "gqa" else 1.0
    _, Hq, Sq, _ = q.shape; Skv = k.shape[2]
    o = torch.zeros_like(q); lse = torch.zeros(1, Hq, Sq, device="cuda")
    s1 = torch.zeros(1, Hq, Skv, device="cuda"); s2 = torch.zeros(1, Hq, Skv, device="cuda")
    ops.attention(q, k, v, o, scale, causal, lse=lse)
    ops.attention_colstats(q, k, lse, scale, causal, s1, s2)
    close(o[0], T(case + "_o"), 2e-2, 1e-2); close(lse[0], T(case + "_lse"), 1e-3, 1e-3)
    close(s1[0], T(case + "_colsum"), 1e-5, 1e-3); close(s2[0], T(case + "_colsumsq"), 1e-5, 1e-3)
    if case == "gqa":
        noise = T("gqa_noise")[None].cuda(); tau = float(G["gqa_tau"])
        lsep = torch.zeros_like(lse); sc = torch.zeros_like(s1)
        ops.attention(q, k, v, o, scale, causal, noise=noise, tau=tau, lse_pert=lsep)
        ops.attention_colstats(q, k, lsep, scale, causal, sc, None, noise=noise, tau=tau)
        close(sc[0], T("gqa_pert_colsum"), 1e-5, 1e-3)
        close(o[0], T("gqa_o"), 2e-2, 1e-2)


def test_oracle_lora_and_gated_mlp_kat():
    close(ref.lora(T("lora_x"), T("lora_w"), T("lora_a"), T("lora_b")), T("lora_o"), 2e-3, 2e-3)
    close(ref.gated_mlp(T("gmlp_x"), T("gmlp_w1"), T("gmlp_w2"), "sigmoid"), T("gmlp_o_sigmoid"), 2e-3, 2e-3)
    close(ref.gated_mlp(T("gmlp_x"), T("gmlp_w1"), T("gmlp_w2"), "silu"), T("gmlp_o_silu"), 2e-3, 2e-3)


@pytest.mark.gpu
def test_hip_lora_and_gated_mlp_kat():
    from triton_amd import modules
    t = dict(X=T("lora_x").cuda(), W=T("lora_w").cuda(), A=T("lora_a").cuda(), B=T("lora_b").cuda())
    t["O"] = torch.zeros(5, 48, dtype=torch.float16, device="cuda")
    mod = modules.get("lora", "linear")
    mod.forward(*[t[n] for n in mod.TENSOR_PARAMS])
    close(t["O"], T("lora_o"), 2e-3, 1e-2)
    for gate in ("sigmoid", "silu"):
        t = dict(X=T("gmlp_x").cuda(), W1=T("gmlp_w1").cuda(), W2=T("gmlp_w2").cuda(), O=torch.zeros(5, 40, dtype=torch.float16, device="cuda"))
        mod = modules.get("gmlp", "linear", gate=gate)
        mod.forward(*[t[n] for n in mod.TENSOR_PARAMS])
        close(t["O"], T("gmlp_o_" + gate), 2e-3, 1e-2)


@pytest.mark.gpu
def test_hip_qknorm_and_projection_kat():
    from triton_amd import modules, ops
    mod = modules.get("qknorm", eps=float(G["qkn_eps"]), scale=0.125)
    t = dict(Q=T("qkn_q")[None].cuda(), K=T("qkn_k")[None].cuda(), V=T("qkn_v")[None].cuda(),
             gamma_q=T("qkn_gq").cuda(), gamma_k=T("qkn_gk").cuda())
    t["O"] = torch.zeros_like(t["Q"])
    mod.forward(*[t[n] for n in mod.TENSOR_PARAMS])
    close(t["O"][0], T("qkn_o"), 2e-2, 1e-2)
    x = T("prj_x").cuda(); n = x.shape[0]
    q = torch.zeros(n, 128, dtype=torch.float16, device="cuda"); k = torch.zeros(n, 64, dtype=torch.float16, device="cuda")
    v = torch.zeros_like(k)
    hm = lambda a: a.view(n, -1, 64).permute(1, 0, 2)
    ops.prenorm_qkv(x, T("prj_gamma").cuda(), T("prj_wq").cuda(), T("prj_wk").cuda(), T("prj_wv").cuda(), hm(q), hm(k), hm(v),
                    float(G["prj_eps"]), True)
    close(q, T("prj_q"), 2e-2, 1e-2); close(k, T("prj_k"), 2e-2, 1e-2); close(v, T("prj_v"), 2e-2, 1e-2)
