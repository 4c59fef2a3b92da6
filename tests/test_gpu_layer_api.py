"""The reference's own Python tests for the layer (src/python/tests/test_layer.py:53-340),
restated against this package: same shapes, same assertions, plus the numeric parity the
reference only checks at 5e-2."""
import pytest
import torch

from helpers import rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dynamic", [False, True])
def test_layer_forward(dynamic):
    from mhc import MHCLayer
    B, n, C = 8, 4, 128
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, use_dynamic_h=dynamic).cuda()
    x = torch.randn(B, n, C, device="cuda")
    out = layer(x)
    assert out.shape == (B, n, C) and out.dtype == torch.float32
    assert not torch.isnan(out).any() and not torch.isinf(out).any()


@pytest.mark.parametrize("dynamic", [False, True])
def test_layer_backward_all_params_get_gradients(dynamic):
    from mhc import MHCLayer
    B, n, C = 4, 4, 64
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, use_dynamic_h=dynamic).cuda()
    x = (torch.randn(B, n, C, device="cuda") + 0.1).requires_grad_(True)
    layer(x).sum().backward()
    assert x.grad is not None and not torch.isnan(x.grad).any()
    for name, p in layer.named_parameters():
        assert p.grad is not None, f"{name} has no gradient"
        assert p.grad.dtype == p.dtype and p.grad.shape == p.shape
        assert not torch.isnan(p.grad).any(), f"{name} has NaN gradient"
        if dynamic and name != "rmsnorm_weight":
            assert p.grad.abs().sum() > 0, f"{name} gradient is zero"


def test_layer_dynamic_matches_naive_small():
    """test_layer.py:145-193 at its own shape (B=2, n=4, C=16, 3 iterations), but at 1e-5."""
    from mhc import MHCLayer
    B, n, C = 2, 4, 16
    torch.manual_seed(42)
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, sinkhorn_iters=3, use_dynamic_h=True).cuda()
    x = torch.randn(B, n, C, device="cuda", requires_grad=True)
    dy = torch.randn(B, n, C, device="cuda")
    out = layer(x)
    # (the reference test uses out.sum(); under that loss the true phi_res gradient is ~0 because
    # the Sinkhorn output's column sums are constant, so a random upstream gradient is used here)
    out.backward(dy)
    p = {k: getattr(layer, k).detach().cpu().float() for k in nm.DYN_PARAM_NAMES if k != "w"}
    p["w"] = layer.rmsnorm_weight.detach().cpu().float()
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x.detach().cpu(), p, dy.cpu(), 3, layer.eps, dtype=torch.float64)
    assert rel_err(out, y_ref) < 1e-5
    assert rel_err(x.grad, g_ref["x"]) < 1e-5
    assert rel_err(layer.phi_res.grad, g_ref["phi_res"]) < 1e-5
    # and the reference's own assertion, at its tolerance, under its loss
    layer.zero_grad()
    x2 = x.detach().clone().requires_grad_(True)
    layer(x2).sum().backward()
    _, g_sum = nm.mhc_dynamic_fwd_bwd(x.detach().cpu(), p, torch.ones(B, n, C), 3, layer.eps, dtype=torch.float64)
    torch.testing.assert_close(x2.grad.cpu().double(), g_sum["x"], rtol=1e-1, atol=1e-1)
    torch.testing.assert_close(layer.phi_res.grad.cpu().double(), g_sum["phi_res"], rtol=1e-1, atol=1e-1)


@pytest.mark.parametrize("dynamic", [False, True])
def test_training_steps_and_batch_sizes(dynamic):
    from mhc import MHCLayer
    n, C = 4, 128
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, use_dynamic_h=dynamic).cuda()
    opt = torch.optim.Adam(layer.parameters(), lr=1e-3)
    x, target = torch.randn(8, n, C, device="cuda"), torch.randn(8, n, C, device="cuda")
    losses = []
    for _ in range(3):
        opt.zero_grad()
        loss = ((layer(x) - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(l == l for l in losses) and losses[-1] < losses[0]
    for B in [1, 4, 16, 32]:
        assert layer(torch.randn(B, n, C, device="cuda")).shape == (B, n, C)


def test_numerical_stability_and_determinism():
    from mhc import MHCLayer
    B, n, C = 8, 4, 128
    for dynamic in (False, True):
        layer = MHCLayer(hidden_dim=C, expansion_rate=n, use_dynamic_h=dynamic).cuda()
        for scale in (100.0, 0.001):
            out = layer(torch.randn(B, n, C, device="cuda") * scale)
            assert not torch.isnan(out).any() and not torch.isinf(out).any()
        x = torch.randn(B, n, C, device="cuda")
        assert torch.equal(layer(x), layer(x))


def test_static_inference_path_matches_training_path():
    from mhc import MHCLayer
    B, n, C = 8, 4, 128
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, use_dynamic_h=False).cuda()
    with torch.no_grad():
        layer.H_res.copy_(torch.randn(n, n))
        layer.H_pre.copy_(torch.randn(n))
    x = torch.randn(B, n, C, device="cuda")
    y_train = layer(x)
    layer.eval()
    with torch.no_grad():
        y_inf = layer(x)
    assert torch.equal(y_train, y_inf)


def test_bf16_input_and_output_dtype_option():
    from mhc import MHCLayer
    B, n, C = 8, 4, 128
    layer = MHCLayer(hidden_dim=C, expansion_rate=n).cuda()
    x = torch.randn(B, n, C, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    y = layer(x)
    assert y.dtype == torch.float32          # the reference's contract
    y.sum().backward()
    assert x.grad.dtype == torch.bfloat16
    layer2 = MHCLayer(hidden_dim=C, expansion_rate=n, output_dtype=torch.bfloat16).cuda()
    assert layer2(x.detach()).dtype == torch.bfloat16


def test_phi_cache_follows_parameter_updates():
    """The concatenated phi is cached between calls and must be rebuilt after an in-place update."""
    from mhc import MHCLayer
    B, n, C = 4, 4, 64
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, alpha_init=1.0).cuda()
    x = torch.randn(B, n, C, device="cuda")
    y0 = layer(x).detach().clone()
    with torch.no_grad():
        layer.phi_res.mul_(-3.0)
    y1 = layer(x).detach()
    assert (y0 - y1).abs().max() > 1e-4


@pytest.mark.parametrize("cache", [False, True])
def test_parameter_updates_always_reach_the_kernels(cache):
    """The gathered copy of phi / bias / alpha is rebuilt on every call by default, so any way of
    writing a parameter is seen (also through `.data`, which does not bump the version counter); with
    the opt-in cache, in-place updates that bump the counter and new tensors at reused addresses are."""
    import gc
    from mhc import MHCLayer, ops
    B, n, C = 4, 4, 64
    x = torch.randn(B, n, C, device="cuda")
    ops.set_param_cache(cache)
    try:
        layer = MHCLayer(hidden_dim=C, expansion_rate=n, alpha_init=1.0).cuda()
        y0 = layer(x).detach().clone()
        assert torch.equal(layer(x).detach(), y0)
        with torch.no_grad():
            layer.b_res.add_(1.0, alpha=1.0).mul_(torch.linspace(-2, 2, n * n, device="cuda").reshape(n, n))
            layer.alpha_res.mul_(-2.0)
        y1 = layer(x).detach().clone()
        assert (y0 - y1).abs().max() > 1e-4
        if not cache:
            layer.phi_res.data.copy_(torch.randn_like(layer.phi_res))   # version counter unchanged
            assert (y1 - layer(x).detach()).abs().max() > 1e-4

        # same shapes, same allocation pattern, different values: the outputs must follow the new values
        outs = []
        for seed in (1, 2):
            del layer
            gc.collect()
            torch.manual_seed(seed)
            layer = MHCLayer(hidden_dim=C, expansion_rate=n, alpha_init=1.0).cuda()
            with torch.no_grad():
                layer.b_res.normal_()
            p = {k: getattr(layer, k).detach().float().cpu() for k in nm.DYN_PARAM_NAMES if k != "w"}
            p["w"] = layer.rmsnorm_weight.detach().float().cpu()
            ref, _ = nm.mhc_dynamic_fwd_bwd(x.cpu(), p, torch.ones(B, n, C), layer.sinkhorn_iters, layer.eps,
                                            dtype=torch.float64)
            y = layer(x).detach().cpu()
            assert rel_err(y, ref) < 1e-5
            outs.append(y)
        assert (outs[0] - outs[1]).abs().max() > 1e-4
    finally:
        ops.set_param_cache(False)


def test_misaligned_views_are_copied_not_refused():
    """A contiguous view whose storage offset is not a multiple of 16 bytes still works."""
    from mhc import MHCLayer
    B, n, C = 3, 4, 64
    layer = MHCLayer(hidden_dim=C, expansion_rate=n).cuda()
    flat = torch.randn(B * n * C + 1, device="cuda")
    x = flat[1:].view(B, n, C)
    assert x.data_ptr() % 16 != 0 and x.is_contiguous()
    assert torch.equal(layer(x), layer(x.clone()))


@pytest.mark.parametrize("dynamic", [False, True])
def test_layer_unusual_inputs(dynamic):
    """Half and double inputs are widened like the reference's .float() (gradients come back in the
    input's dtype), views that are not contiguous are accepted, and a graph kept alive can be
    differentiated twice with the same result."""
    from mhc import MHCLayer
    B, n, C = 5, 4, 96
    torch.manual_seed(3)
    layer = MHCLayer(hidden_dim=C, expansion_rate=n, use_dynamic_h=dynamic).cuda()
    base = torch.randn(B, n, C, device="cuda")
    y0 = layer(base)
    for dt in (torch.float16, torch.float64):
        x = base.to(dt).requires_grad_(True)
        y = layer(x)
        assert y.dtype == torch.float32
        y.sum().backward()
        assert x.grad.dtype == dt and x.grad.shape == x.shape
        assert rel_err(y, layer(x.detach().float())) < 1e-6
    xt = base.transpose(0, 1).contiguous().transpose(0, 1)   # same values, strides of [n, B, C]
    assert not xt.is_contiguous()
    assert torch.equal(layer(xt), y0)
    x = base.clone().requires_grad_(True)
    y = layer(x)
    g1, = torch.autograd.grad(y, x, torch.ones_like(y), retain_graph=True)
    g2, = torch.autograd.grad(y, x, torch.ones_like(y))
    assert torch.equal(g1, g2)
    layer.eval()
    with torch.no_grad():
        assert rel_err(layer(base), y0) < 1e-6   # inference path: same numbers, nothing saved
