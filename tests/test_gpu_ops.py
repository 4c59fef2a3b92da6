"""Stand-alone operators (reference src/python/tests/test_ops.py, src/csrc/tests/test_sinkhorn_knopp.cu,
test_rmsnorm*.cu) through the C ABI, against the oracle restatements."""
import pytest
import torch

from helpers import rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu


def test_sinkhorn_knopp_doubly_stochastic():
    from mhc import sinkhorn_knopp
    torch.manual_seed(42)
    inp = torch.rand(32, 32, device="cuda") + 0.1
    out = sinkhorn_knopp(inp, num_iters=20)
    assert torch.allclose(out.sum(1), torch.ones(32, device="cuda"), atol=1e-5)
    assert torch.allclose(out.sum(0), torch.ones(32, device="cuda"), atol=1e-5)
    assert (out >= 0).all()


@pytest.mark.parametrize("shape,iters", [((32, 32), 10), ((64, 64), 20), ((4, 4), 20), ((5, 9), 7),
                                         ((3, 16, 16), 10), ((128, 128), 5), ((2, 8, 8), 20),
                                         ((70000, 4, 4), 20), ((3000, 32, 32), 3), ((7, 128, 3), 1024),
                                         ((4, 3, 100), 200), ((2, 64, 128), 60),
                                         # square matrices up to 8 x 8 with at most 96 iterations: the in-register kernel
                                         ((9, 3, 3), 20), ((5, 7, 7), 96), ((1030, 8, 8), 20), ((6, 5, 5), 0), ((3, 2, 2), 1),
                                         ((3, 8, 8), 97), ((7, 1, 1), 5)])
def test_sinkhorn_knopp_forward_backward_vs_oracle(shape, iters):
    from mhc import sinkhorn_knopp
    g = torch.Generator().manual_seed(1)
    inp = torch.rand(*shape, generator=g) + 0.1
    go = torch.randn(*shape, generator=g)
    ref_in = inp.double().requires_grad_(True)
    ref = nm.sinkhorn_knopp_plain(ref_in, iters, 1e-8)
    ref.backward(go.double())
    x = inp.cuda().requires_grad_(True)
    out = sinkhorn_knopp(x, num_iters=iters, eps=1e-8)
    out.backward(go.cuda())
    assert rel_err(out, ref.detach()) < 1e-5
    assert rel_err(x.grad, ref_in.grad) < 1e-4


def test_sinkhorn_knopp_stability_and_zero_rows():
    from mhc import sinkhorn_knopp
    for inp in (torch.rand(32, 32, device="cuda") * 1000, torch.rand(32, 32, device="cuda") * 1e-6 + 1e-8):
        out = sinkhorn_knopp(inp, num_iters=50)
        assert not torch.isnan(out).any() and not torch.isinf(out).any()
    z = torch.zeros(4, 4, device="cuda")
    assert torch.equal(sinkhorn_knopp(z, num_iters=3), z)   # thresholded division: no 0/0


@pytest.mark.parametrize("rows,C", [(8, 128), (128, 4096), (16, 64), (5, 100), (3, 100000), (70000, 64), (1, 1),
                                    # rows in registers: one wave per row (1, 2, 4 pieces per thread), a workgroup per row
                                    # (2, 4, 8, 16 pieces), ragged last pieces, row counts off the rows-per-workgroup grid;
                                    # 32768 channels: row kernel forward, generic kernel backward
                                    (5, 1024), (1030, 2048), (7, 8192), (3, 16384), (2, 32768), (9, 4104), (6, 520),
                                    (2500, 264)])
def test_rmsnorm_forward_backward_vs_oracle(rows, C):
    """bf16 operator as in the reference (test_rmsnorm.cu tolerance 1e-2, backward 2e-2)."""
    from mhc import rmsnorm
    g = torch.Generator().manual_seed(2)
    inp = (torch.randn(rows, C, generator=g) * 0.5).bfloat16()
    w = (1 + 0.2 * torch.randn(C, generator=g)).bfloat16()
    go = torch.randn(rows, C, generator=g).bfloat16()
    xr, wr = inp.float().requires_grad_(True), w.float().requires_grad_(True)
    nm.rmsnorm(xr, wr, 1e-5).backward(go.float())
    x, wd = inp.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    out = rmsnorm(x, wd)
    assert out.shape == (rows, C) and out.dtype == torch.bfloat16
    out.backward(go.cuda())
    assert rel_err(out.float(), nm.rmsnorm(inp.float(), w.float(), 1e-5)) < 1e-2
    assert rel_err(x.grad.float(), xr.grad) < 2e-2
    assert rel_err(wd.grad.float(), wr.grad) < 2e-2


@pytest.mark.parametrize("rows,C", [(16, 64), (37, 1028), (9, 8192), (1100, 260), (3, 12288), (5, 1023)])
def test_rmsnorm_fp32_through_c_abi(rows, C):
    from mhc.ops import RMSNormFunction
    g = torch.Generator().manual_seed(3)
    inp = torch.randn(rows, C, generator=g)
    w = 1 + 0.2 * torch.randn(C, generator=g)
    go = torch.randn(rows, C, generator=g)
    dx_ref, dw_ref = nm.rmsnorm_backward_ref(go.double(), inp.double(), w.double(), 1e-5)
    x, wd = inp.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    out = RMSNormFunction.apply(x, wd, 1e-5)
    out.backward(go.cuda())
    assert rel_err(out, nm.rmsnorm(inp.double(), w.double(), 1e-5)) < 1e-6
    assert rel_err(x.grad, dx_ref) < 1e-5 and rel_err(wd.grad, dw_ref) < 1e-5
