"""Workload shapes: the five prefill configurations this build is measured on, and the
reference's own decode-append shapes (convert_eval_rms.py:33-60).  Peak figures for rooflines."""
from __future__ import annotations

HBM_PEAK_GBPS = 8000.0            # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2516.6     # MI355X dense fp16: 256 CU x 2.4 GHz x 4096 flop/clk/CU

LLAMA = dict(n_heads=32, n_kv_heads=8, head_dim=128, hidden=4096)      # Llama3-8B attention shape
FALCON = dict(n_heads=71, n_kv_heads=1, head_dim=64, hidden=4544)      # Falcon-7B attention shape

RMSNORM = dict(rows=4096, cols=4096, eps=1e-5)
VANILLA = dict(batch=1, seq=4096, **LLAMA)
PRENORM = dict(batch=1, seq=2048, eps=1e-5, **LLAMA)
QKNORM = dict(batch=1, seq=2048, eps=1e-5, **FALCON)
KEYFORMER = dict(batch=1, seq=4096, tau=1.0, noise_seed=1234, **LLAMA)
ROCO = dict(batch=1, seq=4096, **LLAMA)

# Reference decode-append shapes: M new tokens, P cached.
DECODE_LLAMA = dict(M=16, N=4096, D=128, H=32, P=1024)
DECODE_FALCON = dict(M=16, N=4544, D=64, H=71, P=1024)


def attn_flops(batch: int, n_heads: int, seq_q: int, seq_kv: int, head_dim: int, causal: bool) -> float:
    """4*B*H*Sq*Skv*D for QK^T and PV together; halved under a causal mask (the convention used for
    every attention figure this build reports)."""
    f = 4.0 * batch * n_heads * seq_q * seq_kv * head_dim
    return f / 2 if causal else f


def rmsnorm_bytes(rows: int, cols: int) -> int:
    """x read once + y written once + gamma, fp16."""
    return 2 * rows * cols * 2 + cols * 2


def qkv_gemm_flops(tokens: int, hidden: int, n_q: int, n_kv: int) -> float:
    return 2.0 * tokens * hidden * (n_q + 2 * n_kv)


def randn_half(shape, gen, mean: float = 0.0, std: float = 1.0):
    """Synthetic fp16 tensor ~ N(mean, std) drawn in fp32 from a seeded generator (the benchmark inputs)."""
    import torch
    return (mean + std * torch.randn(shape, generator=gen, dtype=torch.float32)).half()
