"""CPU restatement of the reference PyTorch path -- TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it.  Nothing under triton_amd/ does.

Every function computes in fp32 from (usually fp16) inputs and rounds the
attention / norm outputs back to the input dtype; key scores stay fp32.  Each
function has "knobs" (scale, causal, eps, gamma, KV-head count, tau, prefix P)
whose neutral setting reproduces the reference class it cites, and whose other
settings give the prefill configurations this build is benchmarked on.

Reference lines restated here (paths are inside the reference repository):
  rmsnorm            ref_attn.py:345-350 (eps + weight form), ref_rms.py:102-103 (bare form)
  attention          ref_rms.py:72-81 (Vanila), ref_rms.py:1454-1477 (batched [B,H,S,D] layout)
  qknorm_attention   ref_rms.py:217-231 (QKNorm: new k normalised, cache prefix not)
  keyformer          ref_rms.py:171-179 (perturbed softmax beside the plain one)
  roco               ref_rms.py:272-280 (column sum and column sum of squares)
  prenorm_block      ref_rms.py:101-127 and convert_eval_rms.py:122-162 (per-head column slices)
  decode_append_*    ref_rms.py:45-83, 101-127, 147-179, 197-231, 249-280 line by line
  seeded inputs      convert_eval_rms.py:170-214 (seed 42, randn.clamp(-1,1)*0.01, noise = randn)

Parity pinning: the reference holds no tests, golden vectors or fixtures for this
path, so each function is pinned by closed forms, invariants, library routines
(F.rms_norm, F.scaled_dot_product_attention) and fp64 brute force on tiny shapes
in tests/test_oracle_*.py.  One statistic the reference does not define -- RoCo's
per-key *mean and standard deviation* (it defines the two sums) -- is stated here
as numpy's mean / std (population) of the probabilities of the queries that can
see the key, and roco_mean_std is held to exactly that on random inputs; there is
no reference formula for it to be at parity with.  The gate of gated_mlp (the
reference names the workload's tensors, not the expression) is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")


# --------------------------------------------------------------------------- RMSNorm
def rmsnorm(x: torch.Tensor, gamma: Optional[torch.Tensor] = None, eps: float = 0.0) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2, -1) + eps) * gamma   (ref_attn.py:348-350).

    gamma=None, eps=0 is the bare form of ref_rms.py:102-103.  fp32 mean-square,
    output rounded to x.dtype.
    """
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    y = xf * torch.rsqrt(var + eps)
    if gamma is not None:
        y = gamma.float() * y
    return y.to(x.dtype)


# --------------------------------------------------------------------------- attention core
def _expand_kv(t: torch.Tensor, n_q_heads: int) -> torch.Tensor:
    """[B,Hkv,S,D] -> [B,Hq,S,D]; query head h reads KV head h // (Hq/Hkv)."""
    hkv = t.shape[1]
    if hkv == n_q_heads:
        return t
    assert n_q_heads % hkv == 0, "query heads must be a multiple of KV heads"
    return t.repeat_interleave(n_q_heads // hkv, dim=1)


def causal_mask(sq: int, skv: int, device=None) -> torch.Tensor:
    """Boolean [sq, skv]; True where query i may see key j: j <= i + (skv - sq).

    With a cached prefix of P = skv - sq keys this is "query i sees keys <= P + i".
    """
    i = torch.arange(sq, device=device).unsqueeze(1)
    j = torch.arange(skv, device=device).unsqueeze(0)
    return j <= i + (skv - sq)


def scores_fp32(q: torch.Tensor, k: torch.Tensor, scale: float, causal: bool) -> torch.Tensor:
    """scale * Q K^T in fp32 with -inf above the causal diagonal.  [B,Hq,Sq,Skv].

    ref_rms.py:77 is the scale=1, causal=False case.
    """
    kf = _expand_kv(k, q.shape[1]).float()
    s = torch.matmul(q.float(), kf.transpose(-1, -2)) * scale
    if causal:
        m = causal_mask(q.shape[-2], k.shape[-2], q.device)
        s = s.masked_fill(~m, NEG_INF)
    return s


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float = 1.0,
              causal: bool = False, return_lse: bool = False):
    """softmax(scale * Q K^T [+ causal]) V.   q [B,Hq,Sq,D]; k,v [B,Hkv,Skv,D].

    ref_rms.py:77-80 (scale=1, causal=False, Hkv=Hq) and ref_rms.py:1466-1473.
    Returns O [B,Hq,Sq,D] in q.dtype (and the natural-log row LSE, fp32, if asked).
    """
    s = scores_fp32(q, k, scale, causal)
    w = torch.softmax(s, dim=-1)
    o = torch.matmul(w, _expand_kv(v, q.shape[1]).float()).to(q.dtype)
    if return_lse:
        return o, torch.logsumexp(s, dim=-1)
    return o


def head_rmsnorm(t: torch.Tensor, gamma: Optional[torch.Tensor], eps: float, start: int = 0) -> torch.Tensor:
    """Per-head RMSNorm over head_dim of rows [start:] along the sequence axis
    (ref_rms.py:217-220); rows before `start` (a cached prefix) pass through."""
    if start <= 0:
        return rmsnorm(t, gamma, eps)
    out = t.clone()
    out[..., start:, :] = rmsnorm(t[..., start:, :], gamma, eps)
    return out


def qknorm_attention(q, k, v, gamma_q=None, gamma_k=None, eps: float = 0.0, scale: float = 1.0,
                     causal: bool = False, k_norm_start: int = 0):
    """Per-head RMSNorm of Q and K over head_dim, then attention (ref_rms.py:217-231).

    The normalised q, k are rounded to fp16 before QK^T as the reference's fp16
    tensors are.  k_norm_start=P leaves a cached prefix un-normalised (ref_rms.py:222).
    """
    qn = head_rmsnorm(q, gamma_q, eps)
    kn = head_rmsnorm(k, gamma_k, eps, k_norm_start)
    return attention(qn, kn, v, scale, causal)


# --------------------------------------------------------------------------- key scores
def keyformer(q, k, v, noise: torch.Tensor, scale: float = 1.0, tau: float = 1.0,
              causal: bool = False, reduce: bool = True):
    """Attention output plus the perturbed-softmax key scores (ref_rms.py:171-179).

    perturb = (scale*QK^T + noise) / tau; perturb_out = softmax(perturb).
    reduce=False returns the un-reduced [B,Hq,Sq,Skv] tensor as the reference class
    does; reduce=True returns its sum over queries, fp32 [B,Hq,Skv], which is what the
    reference's generated kernel stores in C_out (keyformer_llama_benchmark.py:79).
    """
    s = scores_fp32(q, k, scale, causal)
    w = torch.softmax(s, dim=-1)
    o = torch.matmul(w, _expand_kv(v, q.shape[1]).float()).to(q.dtype)
    pert = (s + noise.float()) / tau           # -inf stays -inf under the mask
    pw = torch.softmax(pert, dim=-1)
    return (o, pw.sum(dim=-2)) if reduce else (o, pw)


def roco(q, k, v, scale: float = 1.0, causal: bool = False):
    """Attention output plus per-key sum_i p_ij and sum_i p_ij^2 (ref_rms.py:272-280).
    Both fp32 [B,Hq,Skv]."""
    s = scores_fp32(q, k, scale, causal)
    w = torch.softmax(s, dim=-1)
    o = torch.matmul(w, _expand_kv(v, q.shape[1]).float()).to(q.dtype)
    return o, w.sum(dim=-2), w.pow(2).sum(dim=-2)


def visible_queries(sq: int, skv: int, causal: bool, device=None) -> torch.Tensor:
    """n_j = number of queries that can see key j (fp32 [skv])."""
    if not causal:
        return torch.full((skv,), float(sq), device=device)
    j = torch.arange(skv, device=device)
    return (sq - (j - (skv - sq)).clamp(min=0)).float()


def roco_mean_std(s1: torch.Tensor, s2: torch.Tensor, sq: int, causal: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """mean_j = s1_j / n_j ; std_j = sqrt(max(s2_j / n_j - mean_j^2, 0)).

    The reference defines only the two sums (ref_rms.py:274-275).  The statistic meant here is numpy's
    mean / std (ddof = 0) of column j of the probability matrix over the rows that can see key j;
    tests/test_oracle_pins.py holds this function to that on random inputs and under uniform attention.
    """
    n = visible_queries(sq, s1.shape[-1], causal, s1.device)
    mean = s1 / n
    return mean, (s2 / n - mean * mean).clamp(min=0).sqrt()


# --------------------------------------------------------------------------- PreNorm block
def qkv_project(x: torch.Tensor, gamma, wq, wk, wv, eps: float, norm: bool = True):
    """Xn = RMSNorm(X) (rounded to fp16), then Q,K,V = Xn @ W (fp32 accumulate, rounded).
    X @ W, not X @ W^T (ref_rms.py:105-107)."""
    xn = rmsnorm(x, gamma, eps) if norm else x
    xf = xn.float()
    return tuple((xf @ w.float()).to(x.dtype) for w in (wq, wk, wv))


def split_heads(t: torch.Tensor, head_dim: int) -> torch.Tensor:
    """[B,S,H*D] -> [B,H,S,D]: head h owns columns h*D:(h+1)*D
    (ref_rms.py:109 view; convert_eval_rms.py:132-138 slices)."""
    b, s, n = t.shape
    return t.view(b, s, n // head_dim, head_dim).permute(0, 2, 1, 3)


def prenorm_block(x, gamma, wq, wk, wv, head_dim: int, eps: float = 0.0, scale: float = 1.0,
                  causal: bool = False) -> torch.Tensor:
    """RMSNorm -> QKV projection -> GQA attention -> token-major [B,S,Hq*D]
    (ref_rms.py:101-127 with the layout of ref_rms.py:1477)."""
    q, k, v = qkv_project(x, gamma, wq, wk, wv, eps)
    o = attention(split_heads(q, head_dim), split_heads(k, head_dim), split_heads(v, head_dim), scale, causal)
    return o.permute(0, 2, 1, 3).reshape(x.shape[0], x.shape[1], -1)


# --------------------------------------------------------------------------- decode-append (reference classes)
def _decode_qkv(X, WQ, WK, WV, D, prenorm: bool):
    """q,k,v = X @ W -> [H,M,D] (ref_rms.py:47-56, 102-117).  Returns fp16-rounded heads."""
    M, N = X.shape
    xin = rmsnorm(X) if prenorm else X
    q, k, v = ((xin.float() @ w.float()).to(X.dtype).view(M, N // D, D).transpose(0, 1) for w in (WQ, WK, WV))
    return q, k, v


def _append(cache: torch.Tensor, new: torch.Tensor, P: int) -> torch.Tensor:
    """cat(cache[:, :P], new) (ref_rms.py:72-73)."""
    return torch.cat([cache[:, :P, :], new.to(cache.dtype)], dim=1)


def decode_append_vanilla(X, WQ, WK, WV, K_cache, V_cache, P: int, D: int, prenorm: bool = False):
    """Vanila.forward / PreNorm.forward (ref_rms.py:45-83 / 101-127).  Returns O [H,M,D].

    The reference then does `.view(M, H*D)` on this head-major result without a
    transpose; callers that want that placement call flatten_head_major, callers
    that want the token-major placement of convert_eval_rms.py:160 call
    flatten_token_major.
    """
    q, k, v = _decode_qkv(X, WQ, WK, WV, D, prenorm)
    kc, vc = _append(K_cache, k, P), _append(V_cache, v, P)
    return attention(q[None], kc[None], vc[None], 1.0, False)[0]


def decode_append_qknorm(X, WQ, WK, WV, K_cache, V_cache, P: int, D: int):
    """QKNorm.forward (ref_rms.py:197-231): q and the *new* k are normalised."""
    q, k, v = _decode_qkv(X, WQ, WK, WV, D, False)
    kc, vc = _append(K_cache, rmsnorm(k), P), _append(V_cache, v, P)
    return attention(rmsnorm(q)[None], kc[None], vc[None], 1.0, False)[0]


def decode_append_keyformer(X, WQ, WK, WV, K_cache, V_cache, noise, P: int, D: int, tau: float = 1.5):
    """KeyFormer.forward (ref_rms.py:147-179): returns O [H,M,D], perturb_out [H,M,P+M]."""
    q, k, v = _decode_qkv(X, WQ, WK, WV, D, False)
    kc, vc = _append(K_cache, k, P), _append(V_cache, v, P)
    o, pw = keyformer(q[None], kc[None], vc[None], noise[None], 1.0, tau, False, reduce=False)
    return o[0], pw[0]


def decode_append_roco(X, WQ, WK, WV, K_cache, V_cache, P: int, D: int):
    """RoCo.forward (ref_rms.py:249-280): returns O [H,M,D], sum [H,P+M], sumsq [H,P+M]."""
    q, k, v = _decode_qkv(X, WQ, WK, WV, D, False)
    kc, vc = _append(K_cache, k, P), _append(V_cache, v, P)
    o, s1, s2 = roco(q[None], kc[None], vc[None], 1.0, False)
    return o[0], s1[0], s2[0]


def flatten_head_major(o_hmd: torch.Tensor) -> torch.Tensor:
    """[H,M,D] -> raw view [M,H*D] as ref_rms.py:81 does (no transpose back)."""
    h, m, d = o_hmd.shape
    return o_hmd.contiguous().view(m, h * d)


def flatten_token_major(o_hmd: torch.Tensor) -> torch.Tensor:
    """[H,M,D] -> [M,H*D] with head h in columns h*D:(h+1)*D (convert_eval_rms.py:160)."""
    h, m, d = o_hmd.shape
    return o_hmd.permute(1, 0, 2).reshape(m, h * d)


# --------------------------------------------------------------------------- seeded inputs
def gumbel_noise(shape, seed: int) -> torch.Tensor:
    """Gumbel(0,1) fp32 generated on the host: g = -log(-log(u)), u ~ U(0,1) from a
    CPU generator, clamped away from 0 and 1.  Passed to both sides of a comparison."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    u = torch.rand(shape, generator=gen, dtype=torch.float32).clamp_(1e-10, 1.0 - 1e-7)
    return -torch.log(-torch.log(u))


def randn_half(shape, gen: torch.Generator, mean: float = 0.0, std: float = 1.0) -> torch.Tensor:
    return (mean + std * torch.randn(shape, generator=gen, dtype=torch.float32)).half()


def reference_recipe(shape, gen: torch.Generator) -> torch.Tensor:
    """randn.clamp(-1,1) * 0.01 in fp16 (convert_eval_rms.py:175-183)."""
    return (torch.randn(shape, generator=gen, dtype=torch.float32).half().clamp(-1, 1) * 0.01).half()


def harmonic_tail(S: int, power: int = 1) -> torch.Tensor:
    """sum_{i>=j} 1/(i+1)^power for j = 0..S-1 in fp64 -- the closed form of the causal
    column sums (power 1) and sums of squares (power 2) under uniform attention (Q = 0)."""
    t = 1.0 / torch.arange(1, S + 1, dtype=torch.float64).pow(power)
    return t.flip(0).cumsum(0).flip(0)


def lora(X: torch.Tensor, W: torch.Tensor, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """O = X W + (X A) B (lora_benchmark.py:41-53; intermediates C = X W, D = X A, E = D B, each an fp16 tensor in
    the reference's drivers): products in fp32 from fp16 inputs, every intermediate rounded to fp16."""
    x = X.float()
    c = (x @ W.float()).half()
    d = (x @ A.float()).half()
    e = (d.float() @ B.float()).half()
    return (c.float() + e.float()).half()


def gated_mlp(X: torch.Tensor, W1: torch.Tensor, W2: torch.Tensor, gate: str = "sigmoid") -> torch.Tensor:
    """O = gate(X W1) * (X W2), gate = sigmoid(c) or c * sigmoid(c) (gmlp_benchmark.py:53-64 names X, W1, W2, O and the
    intermediates C1, C1_exp, C2; NodeType.py:21 has the sigmoid operator).
    PARITY UNPINNED beyond its parts: the IR that combines these tensors is not in the reference's tree, so which
    gate the reference evaluates cannot be read off it; each part is a documented torch primitive."""
    x = X.float()
    c1 = (x @ W1.float()).half().float()
    c2 = (x @ W2.float()).half().float()
    g = torch.sigmoid(c1)
    if gate == "silu":
        g = c1 * g
    elif gate != "sigmoid":
        raise ValueError(gate)
    return (g * c2).half()
