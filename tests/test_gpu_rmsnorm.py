"""GPU parity: trn_rmsnorm_f16 (through the C ABI) against the CPU oracle.
Tolerance: 1e-3 relative (fp16 output rounding is 4.9e-4)."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu
RTOL = 1e-3


def _check(y_gpu, want):
    got = y_gpu.float().cpu(); want = want.float()
    err = (got - want).abs()
    assert (err <= RTOL * want.abs() + 1e-6).all(), f"max rel err {(err / want.abs().clamp(min=1e-6)).max()}"


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (16, 4096), (16, 4544), (1, 8), (37, 64), (129, 128),
                                       (5, 520), (3, 8192), (2, 16384), (0, 64)])
@pytest.mark.parametrize("with_gamma", [True, False])
def test_rmsnorm_parity(rows, cols, with_gamma):
    from triton_amd import ops
    g = torch.Generator().manual_seed(42)
    x = ref.randn_half((rows, cols), g)
    gamma = ref.randn_half((cols,), g, 1.0, 0.02) if with_gamma else None
    eps = 1e-5 if with_gamma else 0.0
    xd = x.cuda(); yd = torch.zeros_like(xd)
    ops.rmsnorm(xd, gamma.cuda() if with_gamma else None, yd, eps)
    torch.cuda.synchronize()
    _check(yd, ref.rmsnorm(x, gamma, eps))


def test_rmsnorm_strided_rows_and_closed_form():
    from triton_amd import ops
    base = torch.zeros(8, 256, dtype=torch.float16, device="cuda")
    x = base[:, :128]                      # row pitch 256, 128 columns
    x.fill_(-3.0)
    y = torch.zeros(8, 256, dtype=torch.float16, device="cuda")[:, 64:192]
    ops.rmsnorm(x, None, y, 0.0)
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), torch.full((8, 128), -1.0).half())


def test_head_rmsnorm_prefix_untouched():
    from triton_amd import ops
    g = torch.Generator().manual_seed(1)
    k = ref.randn_half((5, 21, 64), g)
    gamma = ref.randn_half((64,), g, 1.0, 0.02)
    kd = k.cuda(); out = kd.clone()
    ops.head_rmsnorm(kd, gamma.cuda(), out, 1e-5, row_start=16)
    torch.cuda.synchronize()
    want = ref.head_rmsnorm(k, gamma, 1e-5, start=16)
    assert torch.equal(out[:, :16].cpu(), k[:, :16])
    _check(out, want)


@pytest.mark.parametrize("rows,cols", [(64, 4096), (33, 520), (7, 16384)])
def test_rmsnorm_in_place_equals_out_of_place(rows, cols):
    """y may be x itself (DecodeQKNorm normalises the new cache rows where they lie): bit-identical to a separate y."""
    from triton_amd import ops
    g = torch.Generator().manual_seed(9)
    x = ref.randn_half((rows, cols), g); gamma = ref.randn_half((cols,), g, 1.0, 0.02).cuda()
    xd = x.cuda(); sep = torch.zeros_like(xd)
    ops.rmsnorm(xd, gamma, sep, 1e-5)
    ops.rmsnorm(xd, gamma, xd, 1e-5)
    torch.cuda.synchronize()
    assert torch.equal(xd, sep)
    _check(xd, ref.rmsnorm(x, gamma.cpu(), 1e-5))


def test_bad_arguments_raise():
    from triton_amd import ops, _lib
    x = torch.zeros(4, 12, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.TrnError):
        ops.rmsnorm(x, None, torch.zeros_like(x), 0.0)        # cols not a multiple of 8
    with pytest.raises(ValueError):
        ops.rmsnorm(x.float(), None, x, 0.0)
