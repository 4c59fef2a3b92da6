"""Activation tensors with more than 2^31 elements: every index has to be computed in 64 bits.
The oracle checks a handful of samples, the last ones included (y and dx of a sample depend on that
sample only); the parameter gradients, which sum over the batch, are checked against the sum of two
half-batch calls (each half below 2^31 elements)."""
import pytest
import torch

from helpers import rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu


def _run(dyn, x, dy, p, T, eps, out_dtype):
    import mhc
    xd = x.detach().requires_grad_(True)
    q = {k: v.detach().clone().requires_grad_(True) for k, v in p.items()}
    if dyn:
        y = mhc.mhc_layer_fused_dynamic(xd, q["w"], q["phi_pre"], q["phi_post"], q["phi_res"], q["alpha_pre"],
                                        q["alpha_post"], q["alpha_res"], q["b_pre"], q["b_post"], q["b_res"],
                                        T, eps, out_dtype, None)
    else:
        y = mhc.mhc_layer_fused(xd, q["w"], q["H_pre"], q["H_post"], q["H_res"], T, eps, out_dtype, None)
    y.backward(dy)
    torch.cuda.synchronize()
    return y.detach(), xd.grad, {k: v.grad.float() for k, v in q.items()}


@pytest.mark.parametrize("B,n,C,dyn,bf16", [
    (220000, 4, 2560, True, True),     # fused forward, channel-sum and slab kernels
    (110000, 8, 2560, True, True),     # 8 x 8 coefficients, matrix-core projection backward + dx kernel
    (40000, 32, 2048, True, True),     # workgroup-wide Sinkhorn, wide projection kernels
    (140000, 4, 4096, False, False),   # static H, float32
])
def test_layer_beyond_2_31_elements(B, n, C, dyn, bf16):
    T, eps = 20, 1e-6
    assert B * n * C > 2 ** 31
    need = 14 * B * n * C * (2 if bf16 else 4)   # activations, gradients, the two half-batch runs, slack
    if torch.cuda.mem_get_info()[0] < need:
        pytest.skip(f"needs {need >> 30} GiB of free device memory")
    act = torch.bfloat16 if bf16 else torch.float32
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(B, n, C, device="cuda", dtype=act, generator=g)
    dy = torch.randn(B, n, C, device="cuda", dtype=act, generator=g)
    p0 = (nm.make_dynamic_inputs if dyn else nm.make_static_inputs)(1, n, C)[3]
    names = nm.DYN_PARAM_NAMES if dyn else nm.STATIC_PARAM_NAMES
    p = {k: torch.as_tensor(p0[k]).to("cuda", act if k == "w" else torch.float32) for k in names}
    if bf16:
        for k in ("phi_pre", "phi_post", "phi_res"):
            p[k] = p[k].bfloat16().float()   # phi is used in bf16 by this tier
    y, dx, gp = _run(dyn, x, dy, p, T, eps, act)

    last_below = 2 ** 31 // (n * C)   # the sample that straddles element 2^31
    idx = torch.tensor([0, 1, 31, 32, B // 2 - 1, B // 2, last_below, last_below + 1, B - 33, B - 2, B - 1],
                       device="cuda")
    pc = {k: v.float().cpu() for k, v in p.items()}
    fn = nm.mhc_dynamic_fwd_bwd if dyn else nm.mhc_static_fwd_bwd
    y_ref, g_ref = fn(x[idx].float().cpu(), pc, dy[idx].float().cpu(), T, eps,
                      dtype=torch.float32 if bf16 else torch.float64)
    tol = 2e-2 if bf16 else 1e-5
    assert rel_err(y[idx].double().cpu(), y_ref.double()) <= tol
    assert rel_err(dx[idx].double().cpu(), torch.as_tensor(g_ref["x"]).double()) <= tol
    if bf16:
        bad = (y[idx].float().cpu() - y_ref).abs() > 2e-2 * y_ref.abs() + 1e-2
        assert not bool(bad.any())

    h = B // 2
    _, dx1, g1 = _run(dyn, x[:h], dy[:h], p, T, eps, act)
    _, dx2, g2 = _run(dyn, x[h:], dy[h:], p, T, eps, act)
    assert rel_err(dx[idx[:4]].double().cpu(), dx1[idx[:4]].double().cpu()) <= tol
    assert rel_err(dx[idx[-3:]].double().cpu(), dx2[idx[-3:] - h].double().cpu()) <= tol
    for k in gp:
        s = (g1[k] + g2[k]).double().cpu()
        e = rel_err(gp[k].double().cpu(), s)
        # float32 sums in a different order; dw comes back in the parameter's dtype
        bar = 1e-2 if (k == "w" and bf16) else (2e-3 if bf16 else 1e-4)
        assert e <= bar, f"d{k}: full batch vs the two halves {e:.2e}"
    del x, dy, y, dx, dx1, dx2
    torch.cuda.empty_cache()   # tens of GB: hand them back before the next test
