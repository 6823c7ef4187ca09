"""Hand-written counterparts of the reference's generated modules.

The reference's code generator emits, per IR candidate, a Python module with three
attributes (TritonGen.py:568-712):

    TENSOR_PARAMS : sorted names of the tensors `forward` takes (intermediates that fuse away
                    are not listed)
    BLOCK_PARAMS  : sorted names of tunable block-size keyword arguments
    forward(*tensors, block_x=16, ...) -> None : launches the kernels on the current stream and
                    writes the outputs in place

and its drivers call `forward(*[tensors[p] for p in TENSOR_PARAMS])`, first eagerly, then on a
side stream, then under graph capture (vanilla_llama_benchmark.py:243-285), sometimes with the
block sizes as keywords (rms_benchmark.py:252) or positionally after the tensors
(convert_eval_rms.py:275-285).  A FusedModule is such an object with the kernels replaced by
libtrinity_hip.so calls: tile shapes are compile-time choices of the HIP kernels, so
BLOCK_PARAMS is empty and any block-size argument is accepted and ignored.

Shape constants that the reference bakes in at code-generation time (M, N, D, H, P and this
build's scale / causal / eps / tau knobs) are constructor arguments here; the tensor shapes
themselves are read from the tensors on every call.

`forward` allocates nothing after its first call for a given set of shapes: the few
intermediates that do not fuse away (row normalisers, the projected Q of the decode-append
form, an fp32 copy of fp16 noise) live in a per-module workspace cache filled on that first,
eager call -- the call the reference's drivers make before capturing a graph.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .. import ops


class FusedModule:
    """Base: the three-attribute protocol plus a shape-keyed workspace cache.

    A module instance is for one stream at a time: its workspaces (projected queries, row normalisers, the split-key
    counters and partial results of the decode attention) are shared by every `forward` of the instance, so two
    forwards of the same instance that overlap on different streams race.  Give concurrent streams an instance each.
    The cache only grows (a captured graph keeps raw pointers into it); `release()` empties it once no captured
    graph of this instance will be replayed again."""

    TENSOR_PARAMS: List[str] = []
    BLOCK_PARAMS: List[str] = []

    def __init__(self) -> None:
        self._ws: Dict[Tuple, torch.Tensor] = {}

    def _workspace(self, name: str, shape, dtype, device) -> torch.Tensor:
        key = (name, tuple(shape), dtype, str(device))
        t = self._ws.get(key)
        if t is None:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError(
                    f"{type(self).__name__}.forward: first call for shapes {tuple(shape)} is inside a graph "
                    "capture; call forward once eagerly first (as the reference's drivers do)")
            t = torch.empty(shape, dtype=dtype, device=device)
            self._ws[key] = t
        return t

    def release(self) -> None:
        """Drop every cached workspace.  Graphs captured from this instance must not be replayed afterwards."""
        self._ws.clear()

    def _split(self, args, kwargs):
        n = len(self.TENSOR_PARAMS)
        if len(args) < n:
            raise TypeError(f"forward expects tensors {self.TENSOR_PARAMS}, got {len(args)} positional arguments")
        for k in kwargs:
            if not k.startswith("block_"):
                raise TypeError(f"forward got an unexpected keyword argument '{k}'")
        return dict(zip(self.TENSOR_PARAMS, args[:n]))     # trailing positionals are block sizes: ignored

    def forward(self, *args, **kwargs) -> None:
        self._run(**self._split(args, kwargs))

    __call__ = forward

    def _run(self, **tensors) -> None:  # pragma: no cover - abstract
        raise NotImplementedError


def _as4(t: torch.Tensor, name: str) -> torch.Tensor:
    """[H,S,D] -> [1,H,S,D]; 4-D passes through."""
    if t.dim() == 3:
        return t.unsqueeze(0)
    if t.dim() != 4:
        raise ValueError(f"{name}: expected [heads, seq, head_dim] or [batch, heads, seq, head_dim], got {tuple(t.shape)}")
    return t


def _scale(scale: Optional[float], head_dim: int) -> float:
    return head_dim ** -0.5 if scale is None else float(scale)


def _noise_fp32(mod: "FusedModule", n4: torch.Tensor) -> torch.Tensor:
    """The noise as the kernels read it: fp32, unit innermost stride, base and every pitch a multiple of 16 bytes
    (they fetch it with 16-byte loads).  The reference's noise is fp16 (convert_eval_rms.py:201) and its key count
    P + M is arbitrary, so anything else is copied into a workspace whose rows are padded to a multiple of 4 floats;
    the padding is never read as a key (the kernels mask by key index, with selects)."""
    ok = (n4.dtype == torch.float32 and n4.stride(3) == 1 and n4.data_ptr() % 16 == 0
          and all(n4.stride(i) % 4 == 0 for i in range(3)))
    if ok:
        return n4
    B, H, Sq, Skv = n4.shape
    pitch = (Skv + 3) // 4 * 4
    buf = mod._workspace("noise32", (B, H, Sq, pitch), torch.float32, n4.device)
    view = buf[..., :Skv]
    view.copy_(n4)
    return view


def _half_io_ok(t: torch.Tensor, shape) -> bool:
    """A caller-owned fp16 statistics tensor that the kernel can write directly."""
    return t.dtype == torch.float16 and t.is_contiguous() and tuple(t.shape) == tuple(shape)


def _half_noise_ok(n3: torch.Tensor) -> bool:
    """fp16 noise [H, M, P+M] that the decode kernel can read as it is (8-byte pieces)."""
    return (n3.dtype == torch.float16 and n3.dim() == 3 and n3.stride(2) == 1 and n3.data_ptr() % 8 == 0
            and n3.stride(0) % 4 == 0 and n3.stride(1) % 4 == 0)


def _store_scores(dst: torch.Tensor, src32: torch.Tensor) -> None:
    """Key scores are produced in fp32; a caller-owned fp16 tensor (the reference allocates every
    tensor as fp16, vanilla_llama_benchmark.py:131-139) receives them rounded."""
    if dst.data_ptr() != src32.data_ptr():
        dst.copy_(src32.view(dst.shape))


# ============================================================================ prefill form
class RMSNorm(FusedModule):
    """X_norm = RMSNorm(X) * gamma   (ref_attn.py:348-350; gamma=None, eps=0: ref_rms.py:102-103)."""
    TENSOR_PARAMS = ["X", "X_norm", "gamma"]

    def __init__(self, eps: float = 1e-5):
        super().__init__()
        self.eps = eps

    def _run(self, X, X_norm, gamma):
        ops.rmsnorm(X.view(-1, X.shape[-1]), gamma, X_norm.view(-1, X.shape[-1]), self.eps)


class Attention(FusedModule):
    """O = softmax(scale * Q K^T [+causal]) V with GQA/MQA (ref_rms.py:77-80, :1466-1473)."""
    TENSOR_PARAMS = ["K", "O", "Q", "V"]

    def __init__(self, scale: Optional[float] = None, causal: bool = True):
        super().__init__()
        self.scale, self.causal = scale, causal

    def _run(self, K, O, Q, V):
        q, k, v, o = _as4(Q, "Q"), _as4(K, "K"), _as4(V, "V"), _as4(O, "O")
        ops.attention(q, k, v, o, _scale(self.scale, q.shape[-1]), self.causal)


class QKNormAttention(FusedModule):
    """Per-head RMSNorm of Q and K over head_dim, then attention (ref_rms.py:217-228).
    K is normalised once into a workspace (it is shared by every query head); the Q norm is
    fused into the attention kernel's prologue."""
    TENSOR_PARAMS = ["K", "O", "Q", "V", "gamma_k", "gamma_q"]

    def __init__(self, scale: Optional[float] = None, causal: bool = True, eps: float = 1e-5):
        super().__init__()
        self.scale, self.causal, self.eps = scale, causal, eps

    def _run(self, K, O, Q, V, gamma_k, gamma_q):
        q, k, v, o = _as4(Q, "Q"), _as4(K, "K"), _as4(V, "V"), _as4(O, "O")
        if not k.is_contiguous():
            raise ValueError("K: expected a contiguous tensor")
        B, Hkv, Skv, D = k.shape
        kn = self._workspace("k_norm", k.shape, k.dtype, k.device)
        ops.head_rmsnorm(k.view(B * Hkv, Skv, D), gamma_k, kn.view(B * Hkv, Skv, D), self.eps)
        ops.attention(q, kn, v, o, _scale(self.scale, D), self.causal, q_norm=True, gamma_q=gamma_q, q_eps=self.eps)


class KeyFormerAttention(FusedModule):
    """Attention plus key scores C_out[h,j] = sum_i softmax_i((scale*QK^T + noise)/tau)[j]
    (ref_rms.py:171-176; reduced over queries as the generated kernel's C_out is,
    keyformer_llama_benchmark.py:79).  Two launches: forward (+ perturbed row normaliser),
    then the column-owner pass."""
    TENSOR_PARAMS = ["C_out", "K", "O", "Q", "V", "noise"]

    def __init__(self, scale: Optional[float] = None, causal: bool = True, tau: float = 1.0):
        super().__init__()
        self.scale, self.causal, self.tau = scale, causal, tau

    def _run(self, C_out, K, O, Q, V, noise):
        q, k, v, o = _as4(Q, "Q"), _as4(K, "K"), _as4(V, "V"), _as4(O, "O")
        B, Hq, Sq, D = q.shape
        Skv = k.shape[2]
        n4 = _noise_fp32(self, _as4(noise, "noise"))
        lsep = self._workspace("lse_pert", (B, Hq, Sq), torch.float32, q.device)
        score = C_out.view(B, Hq, Skv) if C_out.dtype == torch.float32 and C_out.is_contiguous() else \
            self._workspace("score32", (B, Hq, Skv), torch.float32, q.device)
        sc = _scale(self.scale, D)
        ops.attention(q, k, v, o, sc, self.causal, noise=n4, tau=self.tau, lse_pert=lsep)
        ops.attention_colstats(q, k, lsep, sc, self.causal, score, None, noise=n4, tau=self.tau)
        _store_scores(C_out, score)


class RoCoAttention(FusedModule):
    """Attention plus per-key statistics of the attention probabilities.  stats='sums' (the reference's form,
    ref_rms.py:274-275): C_out1 = column sum, C_out2 = column sum of squares.  stats='mean_std': C_out1 = mean and
    C_out2 = population standard deviation over the queries that can see the key, formed from the two sums in the
    statistics kernel's epilogue."""
    TENSOR_PARAMS = ["C_out1", "C_out2", "K", "O", "Q", "V"]

    def __init__(self, scale: Optional[float] = None, causal: bool = True, stats: str = "sums"):
        super().__init__()
        if stats not in ("sums", "mean_std"):
            raise ValueError("stats: expected 'sums' or 'mean_std'")
        self.scale, self.causal, self.stats = scale, causal, stats

    def _run(self, C_out1, C_out2, K, O, Q, V):
        q, k, v, o = _as4(Q, "Q"), _as4(K, "K"), _as4(V, "V"), _as4(O, "O")
        B, Hq, Sq, D = q.shape
        Skv = k.shape[2]
        lse = self._workspace("lse", (B, Hq, Sq), torch.float32, q.device)
        outs = []
        for i, c in enumerate((C_out1, C_out2)):
            outs.append(c.view(B, Hq, Skv) if c.dtype == torch.float32 and c.is_contiguous() else
                        self._workspace(f"stat32_{i}", (B, Hq, Skv), torch.float32, q.device))
        sc = _scale(self.scale, D)
        ops.attention(q, k, v, o, sc, self.causal, lse=lse)
        if self.stats == "sums":
            ops.attention_colstats(q, k, lse, sc, self.causal, outs[0], outs[1])
        else:
            ops.attention_col_mean_std(q, k, lse, sc, self.causal, outs[0], outs[1])
        _store_scores(C_out1, outs[0]); _store_scores(C_out2, outs[1])


class PreNormBlock(FusedModule):
    """O = Attention(RMSNorm(X) Wq, RMSNorm(X) Wk, RMSNorm(X) Wv), token-major in and out
    (ref_rms.py:101-127 with the layout of ref_rms.py:1477).  X [B,S,hidden], O [B,S,Hq*D].
    Two launches: the RMSNorm-fused projection GEMM writes Q/K/V token-major into a workspace,
    attention reads them as strided [B,H,S,D] views and writes O token-major."""
    TENSOR_PARAMS = ["O", "WK", "WQ", "WV", "X", "gamma"]

    def __init__(self, head_dim: int = 128, scale: Optional[float] = None, causal: bool = True,
                 eps: float = 1e-5, norm: bool = True):
        super().__init__()
        self.head_dim, self.scale, self.causal, self.eps, self.norm = head_dim, scale, causal, eps, norm

    def _run(self, O, WK, WQ, WV, X, gamma):
        D = self.head_dim
        x3 = X if X.dim() == 3 else X.unsqueeze(0)
        o3 = O if O.dim() == 3 else O.unsqueeze(0)
        B, S, K = x3.shape
        nq, nkv = WQ.shape[1], WK.shape[1]
        if not x3.is_contiguous() or not o3.is_contiguous():
            raise ValueError("X, O: expected contiguous tensors")
        qkv = self._workspace("qkv", (B * S, nq + 2 * nkv), X.dtype, X.device)
        qb, kb, vb = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
        hm = lambda t, n: t.view(B * S, n // D, D).permute(1, 0, 2)          # [head, token, D] view
        ops.prenorm_qkv(x3.view(B * S, K), gamma, WQ, WK, WV, hm(qb, nq), hm(kb, nkv), hm(vb, nkv), self.eps, self.norm)
        b4 = lambda t, n: t.view(B, S, n // D, D).permute(0, 2, 1, 3)        # [B, H, S, D] view
        ops.attention(b4(qb, nq), b4(kb, nkv), b4(vb, nkv), b4(o3, nq), _scale(self.scale, D), self.causal)


# ============================================================================ decode-append form
class _DecodeAppend(FusedModule):
    """Common part of the reference's own problem form (ref_rms.py:45-83): M new tokens X [M,N] are
    projected with WQ/WK/WV [N,N]; K and V rows are appended in place at rows P..P+M of the
    [H,P+M,D] caches (convert_eval_rms.py:146-147); every query then attends to all P+M keys with
    no mask and no scale.  O2 [M,N]: o_layout='token_major' puts head h of token m at O2[m, h*D:(h+1)*D], as the
    generated kernels do (convert_eval_rms.py:160); 'head_major' fills O2's memory as [H,M,D], which is what the
    reference classes' `output.view(M, H*D)` of the head-major product leaves there (ref_rms.py:80-81)."""

    def __init__(self, head_dim: int, prenorm: bool = False, scale: float = 1.0, causal: bool = False,
                 o_layout: str = "token_major"):
        super().__init__()
        if o_layout not in ("token_major", "head_major"):
            raise ValueError("o_layout: expected 'token_major' or 'head_major'")
        self.head_dim, self.prenorm, self.scale, self.causal, self.o_layout = head_dim, prenorm, scale, causal, o_layout

    def _project(self, X, WQ, WK, WV, K_cache, V_cache):
        M, N = X.shape
        D = self.head_dim
        H, PM, _ = K_cache.shape
        P = PM - M
        if H * D != N or P < 0 or K_cache.shape != V_cache.shape or K_cache.shape[2] != D:
            raise ValueError(f"inconsistent shapes: X {tuple(X.shape)}, caches {tuple(K_cache.shape)}, head_dim {D}")
        q = self._workspace("q", (H, M, D), X.dtype, X.device)
        ops.prenorm_qkv(X, None, WQ, WK, WV, q, K_cache[:, P:], V_cache[:, P:], 0.0, self.prenorm)
        return q, P

    def _o_view(self, O2, H, M, D):
        """[1,H,M,D] view of O2's memory in the module's output placement."""
        if self.o_layout == "head_major":
            return O2.view(H, M, D).unsqueeze(0)
        return O2.view(M, H, D).permute(1, 0, 2).unsqueeze(0)

    def _attend(self, q, K_cache, V_cache, O2, **kw):
        """Attention of the M new queries over the whole cache, with a workspace (allocated and zeroed once per shape;
        every call leaves its counters at zero again) so that the keys of a head can be split over several workgroups."""
        H, M, D = q.shape
        o = self._o_view(O2, H, M, D)
        nbytes = ops.attention_workspace_bytes(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal)
        ops.attention(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal,
                      workspace=self._split_ws(nbytes, q.device), **kw)

    def _split_ws(self, nbytes: int, device):
        """The split-key workspace (zeroed once, on the cold call that allocates it; the kernels leave its counters at
        zero), or None when the library would not split this problem."""
        if not nbytes:
            return None
        key = ("attn_ws", (nbytes,), torch.uint8, str(device))
        fresh = key not in self._ws
        ws = self._workspace("attn_ws", (nbytes,), torch.uint8, device)
        if fresh:
            ws.zero_()
        return ws


class DecodeVanilla(_DecodeAppend):
    """Vanila.forward / PreNorm.forward (ref_rms.py:45-83 / 101-127)."""
    TENSOR_PARAMS = ["K_cache", "O2", "V_cache", "WK", "WQ", "WV", "X"]

    def _run(self, K_cache, O2, V_cache, WK, WQ, WV, X):
        q, _ = self._project(X, WQ, WK, WV, K_cache, V_cache)
        self._attend(q, K_cache, V_cache, O2)


class DecodeQKNorm(_DecodeAppend):
    """QKNorm.forward (ref_rms.py:197-231): q and the newly appended k rows are normalised
    (no eps, no weight); the cached prefix is used as stored."""
    TENSOR_PARAMS = ["K_cache", "O2", "V_cache", "WK", "WQ", "WV", "X"]

    def _run(self, K_cache, O2, V_cache, WK, WQ, WV, X):
        q, P = self._project(X, WQ, WK, WV, K_cache, V_cache)
        H, M, D = q.shape
        ops.head_rmsnorm(K_cache, None, K_cache, 0.0, row_start=P)          # in place, rows P.. only
        self._attend(q, K_cache, V_cache, O2, q_norm=True, gamma_q=None, q_eps=0.0)


class DecodeKeyFormer(_DecodeAppend):
    """KeyFormer.forward (ref_rms.py:147-179).  reduce=True: the perturbed probabilities summed over the M queries
    into C_out [H,P+M] as the generated kernel does (keyformer_llama_benchmark.py:79).  reduce=False: C_out is the
    un-reduced perturb_out [H,M,P+M] that the reference class returns (ref_rms.py:174-179); M <= 32."""
    TENSOR_PARAMS = ["C_out", "K_cache", "O2", "V_cache", "WK", "WQ", "WV", "X", "noise"]

    def __init__(self, head_dim: int, tau: float = 1.5, reduce: bool = True, **kw):
        super().__init__(head_dim, **kw)
        self.tau, self.reduce = tau, reduce

    def _run(self, C_out, K_cache, O2, V_cache, WK, WQ, WV, X, noise):
        q, _ = self._project(X, WQ, WK, WV, K_cache, V_cache)
        H, M, D = q.shape
        PM = K_cache.shape[1]
        lsep = self._workspace("lse_pert", (1, H, M), torch.float32, X.device)
        o = self._o_view(O2, H, M, D)
        # few heads on a long cache: keys split over workgroups, the key scores as a second launch (fp32 on the way)
        split = ops.attention_stats_workspace_bytes(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal) \
            if self.reduce else 0
        if not split and self.reduce and M <= 32 and _half_io_ok(C_out, (H, PM)) and _half_noise_ok(noise):
            # everything fp16 as the reference's drivers allocate it: one launch, no copies on the side
            ops.attention_with_stats_half(q[None], K_cache[None], V_cache[None], self._o_view(O2, H, M, D), self.scale,
                                          self.causal, C_out.view(1, H, PM), None, noise=noise[None], tau=self.tau,
                                          lse_pert=lsep)
            return
        n4 = _noise_fp32(self, noise[None])
        shape = (1, H, PM) if self.reduce else (1, H, M, PM)
        if C_out.numel() != H * PM * (1 if self.reduce else M):
            raise ValueError(f"C_out {tuple(C_out.shape)}: expected {shape[1:]}")
        score = C_out.view(shape) if C_out.dtype == torch.float32 and C_out.is_contiguous() else \
            self._workspace("score32", shape, torch.float32, X.device)
        if self.reduce:
            # one launch up to 32 new tokens (the key scores are a second sweep inside the attention kernel), two beyond
            ops.attention_with_stats(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal,
                                     score, None, noise=n4, tau=self.tau, lse_pert=lsep,
                                     workspace=self._split_ws(split, X.device))
        else:
            ops.attention_with_probs(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal,
                                     score, noise=n4, tau=self.tau, lse_pert=lsep)
        _store_scores(C_out, score)


class DecodeRoCo(_DecodeAppend):
    """RoCo.forward (ref_rms.py:249-280): C_out1 = weights.sum(dim=1), C_out2 = weights.pow(2).sum(dim=1)."""
    TENSOR_PARAMS = ["C_out1", "C_out2", "K_cache", "O2", "V_cache", "WK", "WQ", "WV", "X"]

    def _run(self, C_out1, C_out2, K_cache, O2, V_cache, WK, WQ, WV, X):
        q, _ = self._project(X, WQ, WK, WV, K_cache, V_cache)
        H, M, D = q.shape
        PM = K_cache.shape[1]
        lse = self._workspace("lse", (1, H, M), torch.float32, X.device)
        o = self._o_view(O2, H, M, D)
        # few heads on a long cache: keys split over workgroups, the statistics as a second launch (fp32 on the way)
        split = ops.attention_stats_workspace_bytes(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal)
        if not split and M <= 32 and _half_io_ok(C_out1, (H, PM)) and _half_io_ok(C_out2, (H, PM)):
            ops.attention_with_stats_half(q[None], K_cache[None], V_cache[None], o, self.scale,
                                          self.causal, C_out1.view(1, H, PM), C_out2.view(1, H, PM), lse=lse)
            return
        outs = []
        for i, c in enumerate((C_out1, C_out2)):
            outs.append(c.view(1, H, PM) if c.dtype == torch.float32 and c.is_contiguous() else
                        self._workspace(f"stat32_{i}", (1, H, PM), torch.float32, X.device))
        ops.attention_with_stats(q[None], K_cache[None], V_cache[None], o, self.scale, self.causal,
                                 outs[0], outs[1], lse=lse, workspace=self._split_ws(split, X.device))
        _store_scores(C_out1, outs[0]); _store_scores(C_out2, outs[1])


class LoRA(FusedModule):
    """O = X W + (X A) B  (lora_benchmark.py:41-53: X [M,N], W [N,P], A [N,R], B [R,P], O [M,P]; the driver's
    intermediates C = X W, D = X A, E = D B stay inside: D is a workspace, C and E never leave the kernels).
    Two launches: {O, D} = X {W, A}, then O = D B + O."""
    TENSOR_PARAMS = ["A", "B", "O", "W", "X"]

    def _run(self, A, B, O, W, X):
        M, N = X.shape
        R, P = B.shape
        if W.shape != (N, P) or A.shape != (N, R) or O.shape != (M, P):
            raise ValueError(f"inconsistent shapes: X {tuple(X.shape)}, W {tuple(W.shape)}, A {tuple(A.shape)}, B {tuple(B.shape)}, O {tuple(O.shape)}")
        d = self._workspace("D", (M, R), X.dtype, X.device)
        ops.linear(X, [W, A], [O, d])
        ops.linear(d, [B], [O], [O])


class GatedMLP(FusedModule):
    """O = gate(X W1) * (X W2)  (gmlp_benchmark.py:53-64: X [M,K], W1, W2 [K,N], O [M,N]; intermediates C1, C1_exp,
    C2).  gate = 'sigmoid' (sigmoid(C1)) or 'silu' (C1 sigmoid(C1)): the reference names the tensors and has a sigmoid
    operator, but the IR that combines them is not in its tree.  One GEMM launch for both products, one for the gate."""
    TENSOR_PARAMS = ["O", "W1", "W2", "X"]

    def __init__(self, gate: str = "sigmoid"):
        super().__init__()
        if gate not in ("sigmoid", "silu"):
            raise ValueError("gate: expected 'sigmoid' or 'silu'")
        self.gate = gate

    def _run(self, O, W1, W2, X):
        M, K = X.shape
        if W1.shape[0] != K or W1.shape != W2.shape or O.shape != (M, W1.shape[1]):
            raise ValueError(f"inconsistent shapes: X {tuple(X.shape)}, W1 {tuple(W1.shape)}, W2 {tuple(W2.shape)}, O {tuple(O.shape)}")
        c2 = self._workspace("C2", tuple(O.shape), X.dtype, X.device)
        ops.linear(X, [W1, W2], [O, c2])            # C1 lands in O and is gated in place
        ops.gate(O, c2, O, self.gate)


PREFILL = {"rms": RMSNorm, "vanilla": Attention, "prenorm": PreNormBlock, "qknorm": QKNormAttention,
           "keyformer": KeyFormerAttention, "roco": RoCoAttention}
DECODE = {"vanilla": DecodeVanilla, "prenorm": lambda **kw: DecodeVanilla(prenorm=True, **kw),
          "qknorm": DecodeQKNorm, "keyformer": DecodeKeyFormer, "roco": DecodeRoCo}


LINEAR = {"lora": LoRA, "gmlp": GatedMLP}


def get(variant: str, form: str = "prefill", **consts) -> FusedModule:
    """Module for `variant` in {'rms','vanilla','prenorm','qknorm','keyformer','roco'} (attention forms) or
    {'lora','gmlp'} (form='linear').
    form='prefill': Q/K/V (or X and weights) given, causal, 1/sqrt(D) scale by default.
    form='decode' : the reference's decode-append problem (needs head_dim=...).
    form='linear' : the reference's LoRA and gated-MLP workloads."""
    table = {"prefill": PREFILL, "decode": DECODE, "linear": LINEAR}.get(form)
    if table is None or variant not in table:
        raise KeyError(f"no module for variant={variant!r} form={form!r}")
    return table[variant](**consts)
