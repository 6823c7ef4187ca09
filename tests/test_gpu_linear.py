"""GPU parity for trn_linear_f16 / trn_gate_f16 and the LoRA / gated-MLP modules built on them, against the CPU
oracle.  Tolerance: fp16 outputs of fp32-accumulated products, atol 2e-3 + rtol 1e-2 at these magnitudes (the kernels'
summation order differs from the oracle's; every intermediate is rounded to fp16 on both sides)."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def close(got, want, atol=2e-3, rtol=1e-2):
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), f"{int(bad.sum())} elements off; max abs err {err.max():.4g}"


# M, N, P, R: the reference's configurations (lora_benchmark.py:545-548) and shapes for each GEMM tiling
LORA_SHAPES = [(16, 1024, 512, 64), (32, 1024, 512, 64), (16, 2048, 1024, 128), (8, 512, 256, 32),
               (1, 64, 8, 8), (200, 264, 320, 24), (2048, 512, 8192, 64)]


@pytest.mark.parametrize("M,N,P,R", LORA_SHAPES)
def test_lora_module_matches_oracle(M, N, P, R):
    from triton_amd import modules
    g = torch.Generator().manual_seed(M + N)
    X, W = ref.randn_half((M, N), g, 0, 0.5), ref.randn_half((N, P), g, 0, 0.05)
    A, B = ref.randn_half((N, R), g, 0, 0.05), ref.randn_half((R, P), g, 0, 0.2)
    mod = modules.get("lora", "linear")
    assert mod.TENSOR_PARAMS == ["A", "B", "O", "W", "X"] and mod.BLOCK_PARAMS == []
    t = dict(A=A.cuda(), B=B.cuda(), O=torch.full((M, P), 7.0, dtype=torch.float16, device="cuda"), W=W.cuda(), X=X.cuda())
    for _ in range(2):                   # O is rewritten, not accumulated into, by a second call
        mod.forward(*[t[n] for n in mod.TENSOR_PARAMS])
    torch.cuda.synchronize()
    close(t["O"], ref.lora(X, W, A, B))


@pytest.mark.parametrize("gate", ("sigmoid", "silu"))
@pytest.mark.parametrize("M,K,N", [(16, 1024, 1024), (8, 520, 264), (300, 264, 1024), (2048, 256, 4096)])
def test_gated_mlp_module_matches_oracle(M, K, N, gate):
    from triton_amd import modules
    g = torch.Generator().manual_seed(K)
    X, W1, W2 = ref.randn_half((M, K), g, 0, 0.5), ref.randn_half((K, N), g, 0, 0.1), ref.randn_half((K, N), g, 0, 0.1)
    mod = modules.get("gmlp", "linear", gate=gate)
    assert mod.TENSOR_PARAMS == ["O", "W1", "W2", "X"]
    t = dict(O=torch.zeros(M, N, dtype=torch.float16, device="cuda"), W1=W1.cuda(), W2=W2.cuda(), X=X.cuda())
    mod.forward(*[t[n] for n in mod.TENSOR_PARAMS])
    torch.cuda.synchronize()
    close(t["O"], ref.gated_mlp(X, W1, W2, gate), atol=4e-3)


def test_linear_strided_rows_three_outputs_and_addend_in_place():
    from triton_amd import ops
    g = torch.Generator().manual_seed(3)
    T, K = 40, 136
    x = ref.randn_half((T, K), g, 0, 0.5)
    ws = [ref.randn_half((K, n), g, 0, 0.1) for n in (72, 8, 200)]
    nan = float("nan")
    xb = torch.full((T + 2, K + 8), nan, dtype=torch.float16, device="cuda"); xb[1:T + 1, :K] = x.cuda()
    outs, bufs = [], []
    for w in ws:
        b = torch.full((T + 2, w.shape[1] + 16), nan, dtype=torch.float16, device="cuda")
        bufs.append(b); outs.append(b[1:T + 1, 8:8 + w.shape[1]])
    add1 = ref.randn_half((T, 8), g, 0, 1.0)
    outs[1].copy_(add1.cuda())                                   # out[1] doubles as its own addend
    ops.linear(xb[1:T + 1, :K], [w.cuda() for w in ws], outs, [None, outs[1], None])
    torch.cuda.synchronize()
    for i, (w, o) in enumerate(zip(ws, outs)):
        want = (x.float() @ w.float()).half()
        if i == 1:
            want = (want.float() + add1.float()).half()
        close(o, want)
    for b, w in zip(bufs, ws):                                   # nothing written outside the views
        mask = torch.ones_like(b, dtype=torch.bool); mask[1:T + 1, 8:8 + w.shape[1]] = False
        assert torch.isnan(b[mask]).all()


def test_linear_and_gate_bad_arguments():
    from triton_amd import ops, _lib
    x = torch.zeros(4, 16, dtype=torch.float16, device="cuda")
    w = torch.zeros(16, 12, dtype=torch.float16, device="cuda")       # 12 columns: not a multiple of 8
    with pytest.raises(_lib.TrnError) as e:
        ops.linear(x, [w], [torch.zeros(4, 12, dtype=torch.float16, device="cuda")])
    assert e.value.status_name == "TRN_E_SHAPE"
    with pytest.raises(ValueError):
        ops.linear(x, [], [])
    with pytest.raises(ValueError):
        ops.gate(x, x, x, "relu")
    with pytest.raises(ValueError):
        ops.linear(x, [torch.zeros(8, 8, dtype=torch.float16, device="cuda")], [torch.zeros(4, 8, dtype=torch.float16, device="cuda")])


def test_lora_under_graph_replay():
    from triton_amd import modules
    g = torch.Generator().manual_seed(1)
    M, N, P, R = 16, 1024, 512, 64
    X, W = ref.randn_half((M, N), g, 0, 0.5), ref.randn_half((N, P), g, 0, 0.05)
    A, B = ref.randn_half((N, R), g, 0, 0.05), ref.randn_half((R, P), g, 0, 0.2)
    t = dict(A=A.cuda(), B=B.cuda(), O=torch.zeros(M, P, dtype=torch.float16, device="cuda"), W=W.cuda(), X=X.cuda())
    mod = modules.get("lora", "linear")
    args = [t[n] for n in mod.TENSOR_PARAMS]
    mod.forward(*args); torch.cuda.synchronize()
    eager = t["O"].clone()
    stream = torch.cuda.Stream(); graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            mod.forward(*args)
    stream.synchronize()
    for i in range(3):
        t["O"].zero_(); torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            graph.replay()
        stream.synchronize()
        assert torch.equal(t["O"], eager), f"replay {i}"
