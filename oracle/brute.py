"""fp64 loop-level brute force of the same arithmetic -- TEST INFRASTRUCTURE ONLY.

Pure-Python / numpy loops written from the mathematical definition (not from
oracle/ref.py's tensor expressions), for tiny shapes.  A dropped term, a wrong
head mapping, a transposed operand or an off-by-one in the causal diagonal in
ref.py shows up as a mismatch against these.

Definitions follow ref_rms.py:77-80 (scores, softmax, weighted sum), :171-174
(perturbed softmax), :274-275 (column sums), ref_attn.py:348-350 (RMSNorm).
"""
from __future__ import annotations

import math

import numpy as np


def rmsnorm(x, gamma=None, eps=0.0):
    x = np.asarray(x, dtype=np.float64)
    out = np.empty_like(x)
    for r in range(x.shape[0]):
        ms = 0.0
        for c in range(x.shape[1]):
            ms += x[r, c] * x[r, c]
        ms /= x.shape[1]
        inv = 1.0 / math.sqrt(ms + eps)
        for c in range(x.shape[1]):
            g = 1.0 if gamma is None else float(gamma[c])
            out[r, c] = x[r, c] * inv * g
    return out


def attention_all(q, k, v, scale=1.0, causal=False, noise=None, tau=1.0):
    """q [Hq,Sq,D], k,v [Hkv,Skv,D] (numpy).  Returns dict with
    o [Hq,Sq,D], lse [Hq,Sq], p [Hq,Sq,Skv], colsum, colsumsq [Hq,Skv],
    and (if noise [Hq,Sq,Skv] given) pert [Hq,Sq,Skv], pert_colsum [Hq,Skv]."""
    q = np.asarray(q, np.float64); k = np.asarray(k, np.float64); v = np.asarray(v, np.float64)
    Hq, Sq, D = q.shape
    Hkv, Skv, _ = k.shape
    group = Hq // Hkv
    o = np.zeros((Hq, Sq, D)); lse = np.zeros((Hq, Sq)); p = np.zeros((Hq, Sq, Skv))
    pert = np.zeros((Hq, Sq, Skv)) if noise is not None else None
    for h in range(Hq):
        hk = h // group
        for i in range(Sq):
            last = (Skv - Sq) + i if causal else Skv - 1       # last visible key
            s = []
            for j in range(last + 1):
                dot = 0.0
                for d in range(D):
                    dot += q[h, i, d] * k[hk, j, d]
                s.append(dot * scale)
            mx = max(s)
            den = sum(math.exp(t - mx) for t in s)
            lse[h, i] = mx + math.log(den)
            for j in range(last + 1):
                p[h, i, j] = math.exp(s[j] - mx) / den
                for d in range(D):
                    o[h, i, d] += p[h, i, j] * v[hk, j, d]
            if noise is not None:
                z = [(s[j] + float(noise[h, i, j])) / tau for j in range(last + 1)]
                mz = max(z)
                dz = sum(math.exp(t - mz) for t in z)
                for j in range(last + 1):
                    pert[h, i, j] = math.exp(z[j] - mz) / dz
    res = dict(o=o, lse=lse, p=p, colsum=p.sum(axis=1), colsumsq=(p * p).sum(axis=1))
    if noise is not None:
        res["pert"] = pert
        res["pert_colsum"] = pert.sum(axis=1)
    return res
