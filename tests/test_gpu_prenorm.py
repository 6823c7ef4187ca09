"""GPU parity: trn_prenorm_qkv_f16 (fused RMSNorm + QKV GEMM) and the whole PreNorm block against the oracle.
Projections are fp16 outputs of a K=hidden fp32-accumulated GEMM: atol 2e-2 / rtol 1e-2."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def close(got, want, atol=2e-2, rtol=1e-2):
    got = got.float().cpu(); want = want.float()
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), f"{int(bad.sum())} off; max abs err {err.max():.4g}"


def weights(g, K, nq, nkv, std=0.02):
    return (ref.randn_half((K, nq), g, 0, std), ref.randn_half((K, nkv), g, 0, std), ref.randn_half((K, nkv), g, 0, std))


@pytest.mark.parametrize("T,K,nq,nkv,D,norm", [(256, 512, 512, 128, 128, True), (130, 520, 192, 64, 64, True),
                                              (16, 4096, 4096, 4096, 128, False), (2048, 4096, 4096, 1024, 128, True),
                                              (1, 64, 64, 64, 64, True), (16, 4544, 4544, 64, 64, True),
                                              # the wide tilings (>= 128 tiles of 256 x 256): ragged tokens and hidden, a
                                              # nearly empty K/V group, no norm -- 256 x 192 tiles (the first three: tiles
                                              # straddle Q | K | V, ragged last tile) and 256 x 256 tiles (the last two)
                                              (1000, 520, 6144, 1024, 128, True), (300, 200, 16384, 64, 64, False),
                                              (900, 264, 8192 + 64, 192, 64, True),
                                              (2048, 200, 6144, 1024, 128, True), (1800, 136, 7168 - 64, 512, 64, False),
                                              # at most 32 tokens: the weight-streaming tiling (four waves split hidden)
                                              (32, 520, 1024, 256, 128, True), (5, 72, 192, 64, 64, True),
                                              (17, 8192, 256, 128, 128, True), (33, 520, 256, 128, 128, True)])
def test_qkv_projection_parity(T, K, nq, nkv, D, norm):
    from triton_amd import ops
    g = torch.Generator().manual_seed(42)
    x = ref.randn_half((T, K), g)
    gamma = ref.randn_half((K,), g, 1.0, 0.02) if norm else None
    wq, wk, wv = weights(g, K, nq, nkv)
    qo = torch.zeros(T, nq, dtype=torch.float16, device="cuda")
    ko = torch.zeros(nkv // D, T, D, dtype=torch.float16, device="cuda")          # head-major
    vo = torch.zeros(T, nkv, dtype=torch.float16, device="cuda")
    ops.prenorm_qkv(x.cuda(), gamma.cuda() if norm else None, wq.cuda(), wk.cuda(), wv.cuda(),
                    qo.view(T, nq // D, D).permute(1, 0, 2), ko, vo.view(T, nkv // D, D).permute(1, 0, 2), 1e-5, norm)
    torch.cuda.synchronize()
    wantq, wantk, wantv = ref.qkv_project(x[None], gamma, wq, wk, wv, 1e-5, norm)
    close(qo, wantq[0]); close(vo, wantv[0])
    close(ko.permute(1, 0, 2).reshape(T, nkv), wantk[0])


def test_projection_into_kv_cache_rows():
    """Decode-append: K, V projections land in rows P..P+M of the [H, P+M, D] caches (ref_rms.py:72-73)."""
    from triton_amd import ops
    M, N, D, P = 16, 512, 64, 40
    H = N // D
    g = torch.Generator().manual_seed(1)
    X = ref.reference_recipe((M, N), g) * 30
    W = [ref.reference_recipe((N, N), g) * 30 for _ in range(3)]
    Kc = ref.reference_recipe((H, P + M, D), g); Vc = ref.reference_recipe((H, P + M, D), g)
    Kd, Vd = Kc.cuda(), Vc.cuda()
    Qd = torch.zeros(H, M, D, dtype=torch.float16, device="cuda")
    ops.prenorm_qkv(X.cuda(), None, W[0].cuda(), W[1].cuda(), W[2].cuda(), Qd, Kd[:, P:], Vd[:, P:], 0.0, False)
    torch.cuda.synchronize()
    q, k, v = ref._decode_qkv(X, *W, D, False)
    assert torch.equal(Kd[:, :P].cpu(), Kc[:, :P]) and torch.equal(Vd[:, :P].cpu(), Vc[:, :P])
    close(Kd[:, P:], k, atol=1e-3); close(Vd[:, P:], v, atol=1e-3); close(Qd, q, atol=1e-3)


@pytest.mark.parametrize("T,K,nq,nkv,D", [(200, 136, 256, 64, 64),         # 128 x 128 tiling
                                         (20, 136, 320, 64, 64),          # weight-streaming tiling
                                         (520, 136, 10240, 512, 128),      # 256 x 192 tiling, tiles straddling Q | K | V
                                         (2048, 136, 6144, 1024, 128)])    # 256 x 256 tiling
def test_projection_reads_and_writes_stay_inside_its_views(T, K, nq, nkv, D):
    """Operands are padded views cut out of NaN-filled buffers, hidden and tokens are ragged: a tile load that strays
    past a row or the end of a view pulls NaN into the product, a store that strays overwrites the NaN padding."""
    from triton_amd import ops
    g = torch.Generator().manual_seed(7)
    x = ref.randn_half((T, K), g); gamma = ref.randn_half((K,), g, 1.0, 0.02)
    wq, wk, wv = weights(g, K, nq, nkv)
    nan = float("nan")

    def padded(t, pad):
        buf = torch.full((t.shape[0] + 3, t.shape[1] + pad), nan, dtype=torch.float16, device="cuda")
        buf[1:1 + t.shape[0], :t.shape[1]] = t.cuda()
        return buf, buf[1:1 + t.shape[0], :t.shape[1]]

    (_, xd), (_, wqd), (_, wkd), (_, wvd) = padded(x, 8), padded(wq, 16), padded(wk, 8), padded(wv, 24)
    outs = []
    for n in (nq, nkv, nkv):
        buf = torch.full((T + 2, n + 8), nan, dtype=torch.float16, device="cuda")
        outs.append((buf, buf[1:1 + T, :n]))
    views = [o[1].unflatten(1, (n // D, D)).permute(1, 0, 2) for o, n in zip(outs, (nq, nkv, nkv))]
    ops.prenorm_qkv(xd, gamma.cuda(), wqd, wkd, wvd, views[0], views[1], views[2], 1e-5, True)
    torch.cuda.synchronize()
    want = ref.qkv_project(x[None], gamma, wq, wk, wv, 1e-5, True)
    for (buf, view), w in zip(outs, want):
        close(view, w[0])
        assert torch.isnan(buf[0]).all() and torch.isnan(buf[T + 1]).all() and torch.isnan(buf[:, view.shape[1]:]).all()
