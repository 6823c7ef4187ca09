"""Operator-level wrappers over the C ABI: argument checks that raise Python exceptions
(so a caller's `try/except` around `forward` behaves as with the reference's generated
modules, vanilla_llama_benchmark.py:303-332), pointer/stride extraction, stream lookup.

Every function writes into caller-owned tensors, launches on torch's current stream and
returns None.  Nothing here allocates device memory.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _dev_half(t: torch.Tensor, name: str) -> None:
    _need(isinstance(t, torch.Tensor), f"{name}: expected a tensor")
    _need(t.is_cuda, f"{name}: expected a GPU tensor, got {t.device}")
    _need(t.dtype == torch.float16, f"{name}: expected float16, got {t.dtype}")
    _need(t.dim() == 0 or t.stride(-1) == 1, f"{name}: innermost stride must be 1")


def _dev_float(t: torch.Tensor, name: str) -> None:
    _need(isinstance(t, torch.Tensor) and t.is_cuda, f"{name}: expected a GPU tensor")
    _need(t.dtype == torch.float32, f"{name}: expected float32, got {t.dtype}")
    _need(t.stride(-1) == 1, f"{name}: innermost stride must be 1")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(t: torch.Tensor):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def rmsnorm(x: torch.Tensor, gamma: Optional[torch.Tensor], y: torch.Tensor, eps: float) -> None:
    """y = RMSNorm(x) over the last axis; x, y [rows, cols] (row stride free), gamma [cols] or None."""
    _dev_half(x, "x"); _dev_half(y, "y")
    _need(x.dim() == 2 and y.shape == x.shape, f"x {tuple(x.shape)} / y {tuple(y.shape)}: expected equal 2-D shapes")
    if gamma is not None:
        _dev_half(gamma, "gamma")
        _need(gamma.shape == (x.shape[1],), f"gamma {tuple(gamma.shape)}: expected ({x.shape[1]},)")
    lib = _lib.load()
    st = lib.trn_rmsnorm_f16(_ptr(x), _ptr(gamma), _ptr(y), 1, x.shape[0], x.shape[1],
                             0, x.stride(0), 0, y.stride(0), 0, float(eps), _stream(x))
    _lib.check("trn_rmsnorm_f16", st)


def head_rmsnorm(x: torch.Tensor, gamma: Optional[torch.Tensor], y: torch.Tensor, eps: float,
                 row_start: int = 0) -> None:
    """Per-head RMSNorm over head_dim of rows [row_start:] of x [heads, seq, head_dim]
    (heads may be a flattened batch*heads axis); other rows of y are left untouched."""
    _dev_half(x, "x"); _dev_half(y, "y")
    _need(x.dim() == 3 and y.shape == x.shape, "x, y: expected equal [heads, seq, head_dim] shapes")
    _need(0 <= row_start <= x.shape[1], "row_start out of range")
    if gamma is not None:
        _dev_half(gamma, "gamma")
        _need(gamma.shape == (x.shape[2],), "gamma: expected (head_dim,)")
    lib = _lib.load()
    st = lib.trn_rmsnorm_f16(_ptr(x), _ptr(gamma), _ptr(y), x.shape[0], x.shape[1] - row_start, x.shape[2],
                             x.stride(0), x.stride(1), y.stride(0), y.stride(1), row_start, float(eps),
                             _stream(x))
    _lib.check("trn_rmsnorm_f16", st)


def _attn_desc(q, k, v, o, scale, causal, q_norm, q_eps, noise, tau) -> _lib.AttnDesc:
    for t, n in ((q, "q"), (k, "k")):
        _dev_half(t, n)
        _need(t.dim() == 4, f"{n}: expected [batch, heads, seq, head_dim], got {tuple(t.shape)}")
    B, Hq, Sq, D = q.shape
    _need(k.shape[0] == B and k.shape[3] == D, f"k {tuple(k.shape)} does not match q {tuple(q.shape)}")
    Hkv, Skv = k.shape[1], k.shape[2]
    d = _lib.AttnDesc()
    d.batch, d.n_q_heads, d.n_kv_heads, d.seq_q, d.seq_kv, d.head_dim = B, Hq, Hkv, Sq, Skv, D
    d.q_stride_b, d.q_stride_h, d.q_stride_s = q.stride(0), q.stride(1), q.stride(2)
    d.k_stride_b, d.k_stride_h, d.k_stride_s = k.stride(0), k.stride(1), k.stride(2)
    if v is not None:
        _dev_half(v, "v"); _dev_half(o, "o")
        _need(v.shape == k.shape, f"v {tuple(v.shape)} must equal k {tuple(k.shape)}")
        _need(o.shape == q.shape, f"o {tuple(o.shape)} must equal q {tuple(q.shape)}")
        d.v_stride_b, d.v_stride_h, d.v_stride_s = v.stride(0), v.stride(1), v.stride(2)
        d.o_stride_b, d.o_stride_h, d.o_stride_s = o.stride(0), o.stride(1), o.stride(2)
    d.scale, d.causal = float(scale), int(bool(causal))
    d.q_norm, d.q_norm_eps = int(bool(q_norm)), float(q_eps)
    if noise is not None:
        if noise.dtype == torch.float16:        # (only trn_attn_fwd_stats_half_f16 takes it; the strides count halfs)
            _dev_half(noise, "noise")
        else:
            _dev_float(noise, "noise")
        _need(tuple(noise.shape) == (B, Hq, Sq, Skv), f"noise {tuple(noise.shape)}: expected {(B, Hq, Sq, Skv)}")
        d.noise_stride_b, d.noise_stride_h, d.noise_stride_s = noise.stride(0), noise.stride(1), noise.stride(2)
    d.tau = float(tau)
    return d


def _row_stat(t: Optional[torch.Tensor], name: str, shape) -> None:
    if t is None:
        return
    _dev_float(t, name)
    _need(tuple(t.shape) == tuple(shape) and t.is_contiguous(), f"{name}: expected contiguous float32 {tuple(shape)}")


_scratch_ready = set()


def _static_scratch_ready(device: torch.device) -> None:
    """The library looks up the address of its static scratch array once per GPU, which is no stream operation and
    must not happen under graph capture: do it on the first eager "static" call on a device (trn_check_device), and
    refuse a first call that arrives while the stream is capturing."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx in _scratch_ready:
        return
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError('workspace="static": make one eager call on this GPU (or call trn_check_device) before capturing')
    with torch.cuda.device(idx):
        _lib.check("trn_check_device", _lib.load().trn_check_device())
    _scratch_ready.add(idx)


def attention(q, k, v, o, scale: float, causal: bool, lse: Optional[torch.Tensor] = None,
              q_norm: bool = False, gamma_q: Optional[torch.Tensor] = None, q_eps: float = 0.0,
              noise: Optional[torch.Tensor] = None, tau: float = 1.0,
              lse_pert: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> None:
    """o = softmax(scale * q k^T [+causal]) v.  q,o [B,Hq,Sq,D]; k,v [B,Hkv,Skv,D] (strided views allowed).
    Optional outputs: lse [B,Hq,Sq] fp32; with noise [B,Hq,Sq,Skv] fp32 also lse_pert.
    workspace: optional zero-initialised uint8 tensor of attention_workspace_bytes(...) bytes (decode shapes with
    few heads then split their keys over several workgroups); the string "static" takes the library's own static
    device array instead (nothing is allocated; one such call at a time per GPU)."""
    d = _attn_desc(q, k, v, o, scale, causal, q_norm, q_eps, noise, tau)
    B, Hq, Sq, _ = q.shape
    _row_stat(lse, "lse", (B, Hq, Sq)); _row_stat(lse_pert, "lse_pert", (B, Hq, Sq))
    if gamma_q is not None:
        _dev_half(gamma_q, "gamma_q")
        _need(gamma_q.shape == (q.shape[3],), "gamma_q: expected (head_dim,)")
    _need(noise is None or lse_pert is not None, "noise given without lse_pert")
    lib = _lib.load()
    if isinstance(workspace, str):
        _need(workspace == "static", 'workspace: a uint8 GPU tensor, None, or "static"')
        _static_scratch_ready(q.device)
        st = lib.trn_attn_fwd_noalloc_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(gamma_q),
                                          _ptr(noise), _ptr(lse_pert), _stream(q))
        _lib.check("trn_attn_fwd_noalloc_f16", st)
        return
    if workspace is not None:
        _need(workspace.is_cuda and workspace.is_contiguous() and workspace.dtype == torch.uint8, "workspace: expected a contiguous uint8 GPU tensor")
        st = lib.trn_attn_fwd_ws_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(gamma_q),
                                     _ptr(noise), _ptr(lse_pert), _ptr(workspace), workspace.numel(), _stream(q))
        _lib.check("trn_attn_fwd_ws_f16", st)
        return
    st = lib.trn_attn_fwd_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(gamma_q),
                              _ptr(noise), _ptr(lse_pert), _stream(q))
    _lib.check("trn_attn_fwd_f16", st)


def attention_kernel_name(q, k, v, o, scale: float, causal: bool, with_noise: bool = False) -> str:
    """Name of the kernel instantiation `attention` launches for these tensors, as a profiler prints it."""
    d = _attn_desc(q, k, v, o, scale, causal, False, 0.0, None, 1.0)
    return _lib.load().trn_attn_fwd_kernel_name(C.byref(d), 1 if with_noise else 0).decode()


def attention_workspace_bytes(q, k, v, o, scale: float, causal: bool) -> int:
    """Bytes of workspace with which `attention` would split the keys of this problem over several workgroups (0: none)."""
    d = _attn_desc(q, k, v, o, scale, causal, False, 0.0, None, 1.0)
    return int(_lib.load().trn_attn_workspace_bytes(C.byref(d)))


def attention_stats_workspace_bytes(q, k, v, o, scale: float, causal: bool) -> int:
    """Bytes of workspace with which `attention_with_stats` would split the keys of this problem over several
    workgroups and run the statistics as a second launch (0: it would not -- one launch is faster)."""
    d = _attn_desc(q, k, v, o, scale, causal, False, 0.0, None, 1.0)
    return int(_lib.load().trn_attn_stats_workspace_bytes(C.byref(d)))


def attention_colstats(q, k, lse, scale: float, causal: bool, out_sum: Optional[torch.Tensor],
                       out_sumsq: Optional[torch.Tensor] = None, noise: Optional[torch.Tensor] = None,
                       tau: float = 1.0) -> None:
    """Column sums (and sums of squares) of exp(t - lse) over the queries that see each key.
    lse [B,Hq,Sq] is the row normaliser matching t (plain, or perturbed when noise is given).
    out_sum / out_sumsq: float32 [B,Hq,Skv]."""
    d = _attn_desc(q, k, None, None, scale, causal, False, 0.0, noise, tau)
    B, Hq, Sq, _ = q.shape
    Skv = k.shape[2]
    _need(lse is not None, "lse is required")
    _row_stat(lse, "lse", (B, Hq, Sq))
    _row_stat(out_sum, "out_sum", (B, Hq, Skv)); _row_stat(out_sumsq, "out_sumsq", (B, Hq, Skv))
    _need(out_sum is not None or out_sumsq is not None, "no output given")
    lib = _lib.load()
    st = lib.trn_attn_colstats_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(lse), _ptr(noise), _ptr(out_sum),
                                   _ptr(out_sumsq), _stream(q))
    _lib.check("trn_attn_colstats_f16", st)


def attention_with_probs(q, k, v, o, scale: float, causal: bool, out_probs: torch.Tensor,
                         out_sum: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                         noise: Optional[torch.Tensor] = None, tau: float = 1.0,
                         lse_pert: Optional[torch.Tensor] = None) -> None:
    """Decode shapes (at most 32 queries per head): o, and the un-reduced probabilities out_probs float32
    [B,Hq,Sq,Skv] -- of the perturbed scores when noise is given (KeyFormer's perturb_out) -- in one launch."""
    d = _attn_desc(q, k, v, o, scale, causal, False, 0.0, noise, tau)
    B, Hq, Sq, _ = q.shape
    Skv = k.shape[2]
    _dev_float(out_probs, "out_probs")
    _need(tuple(out_probs.shape) == (B, Hq, Sq, Skv) and out_probs.is_contiguous(), f"out_probs: expected contiguous float32 {(B, Hq, Sq, Skv)}")
    _row_stat(lse, "lse", (B, Hq, Sq)); _row_stat(lse_pert, "lse_pert", (B, Hq, Sq)); _row_stat(out_sum, "out_sum", (B, Hq, Skv))
    _need(noise is None or lse_pert is not None, "noise requires lse_pert")
    st = _lib.load().trn_attn_fwd_probs_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(noise),
                                            _ptr(lse_pert), _ptr(out_probs), _ptr(out_sum), _stream(q))
    _lib.check("trn_attn_fwd_probs_f16", st)


def attention_col_mean_std(q, k, lse, scale: float, causal: bool, out_mean: torch.Tensor, out_std: torch.Tensor) -> None:
    """Per-key mean and population standard deviation of the attention probabilities exp(scale*q k^T - lse) over the
    queries that can see the key (RoCo's statistics in that form).  out_mean, out_std: float32 [B,Hq,Skv]."""
    d = _attn_desc(q, k, None, None, scale, causal, False, 0.0, None, 1.0)
    B, Hq, Sq, _ = q.shape
    Skv = k.shape[2]
    _need(lse is not None and out_mean is not None and out_std is not None, "lse, out_mean and out_std are required")
    _row_stat(lse, "lse", (B, Hq, Sq))
    _row_stat(out_mean, "out_mean", (B, Hq, Skv)); _row_stat(out_std, "out_std", (B, Hq, Skv))
    st = _lib.load().trn_attn_colmeanstd_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(lse), _ptr(out_mean), _ptr(out_std), _stream(q))
    _lib.check("trn_attn_colmeanstd_f16", st)


def attention_with_stats(q, k, v, o, scale: float, causal: bool, out_sum: Optional[torch.Tensor],
                         out_sumsq: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                         noise: Optional[torch.Tensor] = None, tau: float = 1.0,
                         lse_pert: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> None:
    """`attention` and `attention_colstats` in one call (one launch with at most 32 queries per head): o, and the
    column sums / sums of squares of the probabilities -- of the perturbed ones when noise is given.  With more than
    32 queries lse (lse_pert with noise) must be given: it carries the row normalisers between the two kernels.
    workspace: optional zero-initialised uint8 tensor of attention_workspace_bytes(...) bytes: few queries on a long
    cache then run with their keys split over workgroups and the statistics as a second launch (lse / lse_pert
    required, as above)."""
    d = _attn_desc(q, k, v, o, scale, causal, False, 0.0, noise, tau)
    B, Hq, Sq, _ = q.shape
    Skv = k.shape[2]
    _row_stat(lse, "lse", (B, Hq, Sq)); _row_stat(lse_pert, "lse_pert", (B, Hq, Sq))
    _row_stat(out_sum, "out_sum", (B, Hq, Skv)); _row_stat(out_sumsq, "out_sumsq", (B, Hq, Skv))
    _need(out_sum is not None or out_sumsq is not None, "no statistics output given")
    if noise is not None:
        _need(lse_pert is not None, "noise requires lse_pert")
    lib = _lib.load()
    if workspace is not None:
        _need(workspace.is_cuda and workspace.is_contiguous() and workspace.dtype == torch.uint8, "workspace: expected a contiguous uint8 GPU tensor")
        st = lib.trn_attn_fwd_stats_ws_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), None, _ptr(noise),
                                           _ptr(lse_pert), _ptr(out_sum), _ptr(out_sumsq), _ptr(workspace), workspace.numel(),
                                           _stream(q))
        _lib.check("trn_attn_fwd_stats_ws_f16", st)
        return
    st = lib.trn_attn_fwd_stats_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), None, _ptr(noise),
                                    _ptr(lse_pert), _ptr(out_sum), _ptr(out_sumsq), _stream(q))
    _lib.check("trn_attn_fwd_stats_f16", st)


def attention_with_stats_half(q, k, v, o, scale: float, causal: bool, out_sum: Optional[torch.Tensor],
                              out_sumsq: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                              noise: Optional[torch.Tensor] = None, tau: float = 1.0,
                              lse_pert: Optional[torch.Tensor] = None) -> None:
    """`attention_with_stats` for at most 32 queries per head with fp16 noise and fp16 statistics, as the reference's
    drivers allocate them: one launch, nothing widened or narrowed on the side."""
    _need(noise is None or noise.dtype == torch.float16, "noise: expected float16")
    d = _attn_desc(q, k, v, o, scale, causal, False, 0.0, noise, tau)
    B, Hq, Sq, _ = q.shape
    Skv = k.shape[2]
    _need(Sq <= 32, f"{Sq} queries per head: the fp16 form is for at most 32")
    _row_stat(lse, "lse", (B, Hq, Sq)); _row_stat(lse_pert, "lse_pert", (B, Hq, Sq))
    for t, n in ((out_sum, "out_sum"), (out_sumsq, "out_sumsq")):
        if t is not None:
            _dev_half(t, n)
            _need(tuple(t.shape) == (B, Hq, Skv) and t.is_contiguous(), f"{n}: expected contiguous float16 {(B, Hq, Skv)}")
    _need(out_sum is not None or out_sumsq is not None, "no statistics output given")
    if noise is not None:
        _need(lse_pert is not None, "noise requires lse_pert")
    lib = _lib.load()
    st = lib.trn_attn_fwd_stats_half_f16(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), None, _ptr(noise),
                                         _ptr(lse_pert), _ptr(out_sum), _ptr(out_sumsq), _stream(q))
    _lib.check("trn_attn_fwd_stats_half_f16", st)


def prenorm_qkv(x: torch.Tensor, gamma: Optional[torch.Tensor], wq, wk, wv, q_out, k_out, v_out,
                eps: float, norm: bool = True) -> None:
    """Q,K,V = RMSNorm(x; gamma, eps) @ W{q,k,v}  (norm=False: x @ W).
    x [T, hidden]; w* [hidden, n_*]; *_out indexed [head, token, head_dim] (any view with unit
    innermost stride: a permuted token-major buffer, a head-major buffer, or rows of a KV cache)."""
    _dev_half(x, "x")
    _need(x.dim() == 2, "x: expected [tokens, hidden]")
    T, K = x.shape
    for w, n in ((wq, "wq"), (wk, "wk"), (wv, "wv")):
        _dev_half(w, n)
        _need(w.dim() == 2 and w.shape[0] == K, f"{n}: expected [hidden={K}, n_out], got {tuple(w.shape)}")
    _need(wk.shape[1] == wv.shape[1], "wk and wv must have the same number of columns")
    D = q_out.shape[-1]
    for o, w, n in ((q_out, wq, "q_out"), (k_out, wk, "k_out"), (v_out, wv, "v_out")):
        _dev_half(o, n)
        _need(o.dim() == 3 and o.shape[1] == T and o.shape[2] == D and o.shape[0] * D == w.shape[1],
              f"{n}: expected [heads, {T}, {D}] with heads*{D} == {w.shape[1]}, got {tuple(o.shape)}")
    if gamma is not None:
        _dev_half(gamma, "gamma")
        _need(gamma.shape == (K,), "gamma: expected (hidden,)")
    lib = _lib.load()
    st = lib.trn_prenorm_qkv_f16(_ptr(x), _ptr(gamma), _ptr(wq), _ptr(wk), _ptr(wv), _ptr(q_out), _ptr(k_out),
                                 _ptr(v_out), T, K, wq.shape[1], wk.shape[1], D, x.stride(0), wq.stride(0),
                                 wk.stride(0), wv.stride(0), q_out.stride(0), q_out.stride(1), k_out.stride(0),
                                 k_out.stride(1), v_out.stride(0), v_out.stride(1), float(eps), int(bool(norm)),
                                 _stream(x))
    _lib.check("trn_prenorm_qkv_f16", st)


def linear(x: torch.Tensor, weights, outs, addends=None) -> None:
    """outs[i] = x @ weights[i] (+ addends[i]) for up to three weight matrices sharing x.  x [T, hidden]; weights[i]
    [hidden, n_i]; outs[i] / addends[i] [T, n_i]; rows may be strided, innermost stride 1; an addend may be its out."""
    _dev_half(x, "x")
    _need(x.dim() == 2, "x: expected [tokens, hidden]")
    T, K = x.shape
    k = len(weights)
    _need(1 <= k <= 3 and len(outs) == k and (addends is None or len(addends) == k), "expected 1-3 weights with as many outputs")
    adds = list(addends) if addends is not None else [None] * k
    for i, (w, o, ad) in enumerate(zip(weights, outs, adds)):
        _dev_half(w, f"weights[{i}]"); _dev_half(o, f"outs[{i}]")
        _need(w.dim() == 2 and w.shape[0] == K, f"weights[{i}]: expected [hidden={K}, n], got {tuple(w.shape)}")
        _need(tuple(o.shape) == (T, w.shape[1]), f"outs[{i}]: expected [{T}, {w.shape[1]}], got {tuple(o.shape)}")
        if ad is not None:
            _dev_half(ad, f"addends[{i}]")
            _need(tuple(ad.shape) == tuple(o.shape) and ad.stride() == o.stride(), f"addends[{i}]: expected the shape and strides of outs[{i}]")
    vps = lambda ts: (C.c_void_p * k)(*[_ptr(t) for t in ts])
    i64 = lambda vs: (C.c_int64 * k)(*vs)
    lib = _lib.load()
    st = lib.trn_linear_f16(_ptr(x), T, K, x.stride(0), k, vps(weights), i64([w.shape[1] for w in weights]),
                            i64([w.stride(0) for w in weights]), vps(outs), i64([o.stride(0) for o in outs]),
                            vps(adds), _stream(x))
    _lib.check("trn_linear_f16", st)


def gate(c1: torch.Tensor, c2: torch.Tensor, out: torch.Tensor, kind: str = "sigmoid") -> None:
    """out = sigmoid(c1) * c2 ("sigmoid") or c1 * sigmoid(c1) * c2 ("silu"), elementwise over [rows, cols] fp16."""
    _need(kind in ("sigmoid", "silu"), "kind: expected 'sigmoid' or 'silu'")
    for t, n in ((c1, "c1"), (c2, "c2"), (out, "out")):
        _dev_half(t, n)
        _need(t.dim() == 2 and tuple(t.shape) == tuple(c1.shape), f"{n}: expected [rows, cols] like c1")
    lib = _lib.load()
    st = lib.trn_gate_f16(_ptr(c1), _ptr(c2), _ptr(out), c1.shape[0], c1.shape[1], c1.stride(0), c2.stride(0),
                          out.stride(0), 1 if kind == "silu" else 0, _stream(c1))
    _lib.check("trn_gate_f16", st)


def calibration_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst <- src with the library's plain streaming copy kernel (measurement yardstick)."""
    _need(src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous(), "expected contiguous GPU tensors")
    nbytes = src.numel() * src.element_size()
    _need(nbytes == dst.numel() * dst.element_size() and nbytes % 16 == 0, "sizes must match and be a multiple of 16 bytes")
    lib = _lib.load()
    _lib.check("trn_calibration_copy", lib.trn_calibration_copy(_ptr(src), _ptr(dst), nbytes, _stream(src)))


def calibration_mfma(operands: torch.Tensor, sink: torch.Tensor, iters: int, n_workgroups: int) -> float:
    """Launch the MFMA-only yardstick kernel; returns the flop count of the launch."""
    _dev_half(operands, "operands"); _dev_float(sink, "sink")
    _need(operands.numel() >= 32768 and operands.is_contiguous(), "operands: need >= 32768 contiguous fp16 values")
    _need(sink.numel() >= n_workgroups * 256, "sink too small")
    lib = _lib.load()
    _lib.check("trn_calibration_mfma", lib.trn_calibration_mfma(_ptr(operands), _ptr(sink), int(iters), int(n_workgroups),
                                                                _stream(operands)))
    return float(n_workgroups) * 4 * iters * 8 * 32768.0
