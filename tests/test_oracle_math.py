"""Pins of the oracle that come from mathematics rather than from the reference's text:
library routines, closed forms, structural identities and finite differences.  CPU only."""
import numpy as np
import pytest
import torch

from helpers import pack_dynamic, rel_err
from oracle import c_oracle, naive_mhc as nm


def test_rmsnorm_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 48, generator=g, dtype=torch.float64)
    w = torch.randn(48, generator=g, dtype=torch.float64)
    ref = torch.nn.functional.rms_norm(x, (48,), w, 1e-5)
    assert rel_err(nm.rmsnorm(x, w, 1e-5), ref) < 1e-14
    assert rel_err(nm.rmsnorm(x, None, 1e-5), torch.nn.functional.rms_norm(x, (48,), None, 1e-5)) < 1e-14


@pytest.mark.parametrize("n", [1, 2, 4, 8])
def test_sinkhorn_uniform_logits_closed_form(n):
    """All-equal logits stay all-equal: the matrix follows the scalar map m -> m/(n m + eps),
    applied twice per iteration."""
    c, T, eps = 0.37, 6, 1e-2
    m = float(np.exp(c))
    for _ in range(2 * T):
        m = m / (n * m + eps)
    out = nm.sinkhorn_knopp_exp(torch.full((n, n), c, dtype=torch.float64), T, eps)
    assert torch.allclose(out, torch.full((n, n), m, dtype=torch.float64), rtol=1e-13, atol=0)


def test_sinkhorn_order_is_row_then_column_with_eps_added():
    """After ONE iteration the column sums are exactly S/(S+eps) with S the column sums of the
    row-normalised matrix, while the row sums are generally not 1: this fails for
    column-then-row order, for eps placed in a max() or for a thresholded division."""
    g = torch.Generator().manual_seed(3)
    L = torch.randn(5, 5, generator=g, dtype=torch.float64)
    eps = 0.05
    E = torch.exp(L)
    R = E / (E.sum(1, keepdim=True) + eps)
    S = R.sum(0)
    out = nm.sinkhorn_knopp_exp(L, 1, eps)
    assert torch.allclose(out.sum(0), S / (S + eps), rtol=1e-13)
    assert (out.sum(1) - 1).abs().max() > 1e-3
    assert torch.allclose(out, R / (S + eps), rtol=1e-13)


def test_sinkhorn_converges_to_doubly_stochastic_and_is_permutation_equivariant():
    g = torch.Generator().manual_seed(4)
    L = torch.randn(3, 8, 8, generator=g, dtype=torch.float64)
    out = nm.sinkhorn_knopp_exp(L, 200, 1e-12)
    assert (out.sum(-1) - 1).abs().max() < 1e-9 and (out.sum(-2) - 1).abs().max() < 1e-9
    pr, pc = torch.randperm(8, generator=g), torch.randperm(8, generator=g)
    out_p = nm.sinkhorn_knopp_exp(L[:, pr][:, :, pc], 7, 1e-6)
    assert torch.allclose(out_p, nm.sinkhorn_knopp_exp(L, 7, 1e-6)[:, pr][:, :, pc], rtol=1e-12)


def test_identity_mapping():
    """M = I and H_post = 0 make the layer the identity (the property mHC is named for)."""
    n, C = 4, 16
    x = torch.randn(3, n, C, dtype=torch.float64)
    H_res = torch.full((n, n), -60.0, dtype=torch.float64) + 60.0 * torch.eye(n, dtype=torch.float64)
    y = nm.mhc_static_forward(x, torch.ones(C, dtype=torch.float64), torch.zeros(n, dtype=torch.float64),
                              torch.full((n,), -60.0, dtype=torch.float64), H_res, 20, 1e-12)
    assert rel_err(y, x) < 1e-10


def test_mix_is_bmm_and_injected_f_is_consistent():
    x, dy, _, p = nm.make_dynamic_inputs(3, 4, 16, phi_std=0.3, alpha=0.8)
    x = x.double()
    p = {k: torch.as_tensor(v).double() for k, v in p.items()}
    y, im = nm.mhc_dynamic_forward(x, p["w"], p["phi_pre"], p["phi_post"], p["phi_res"], p["alpha_pre"],
                                   p["alpha_post"], p["alpha_res"], p["b_pre"], p["b_post"], p["b_res"],
                                   5, 1e-6, return_intermediates=True)
    ref = torch.bmm(im.M, x) + im.H_post[:, :, None] * im.f[:, None, :]
    assert rel_err(y, ref) < 1e-14
    y2 = nm.mhc_dynamic_forward(x, p["w"], p["phi_pre"], p["phi_post"], p["phi_res"], p["alpha_pre"],
                                p["alpha_post"], p["alpha_res"], p["b_pre"], p["b_post"], p["b_res"],
                                5, 1e-6, f_inject=im.f)
    assert rel_err(y2, y) < 1e-15
    # P is the plain matmul of the normalised rows with phi_concat^T
    phi, _, _ = pack_dynamic(p)
    xn = torch.nn.functional.rms_norm(x.reshape(3, -1), (64,), None, 1e-6)
    assert rel_err(im.P, xn @ phi.t()) < 1e-13


def test_dynamic_with_zero_alpha_is_the_static_layer():
    g = torch.Generator().manual_seed(9)
    B, n, C = 3, 4, 16
    x, dy, _, p = nm.make_dynamic_inputs(B, n, C)
    p["alpha_pre"] = p["alpha_post"] = p["alpha_res"] = torch.tensor(0.0)
    p["b_pre"] = torch.randn(n, generator=g)
    p["b_post"] = torch.randn(n, generator=g)
    p["b_res"] = torch.randn(n, n, generator=g)
    p["w"] = torch.randn(C, generator=g)
    yd, gd = nm.mhc_dynamic_fwd_bwd(x, p, dy, 20, 1e-6, dtype=torch.float64)
    ps = dict(w=p["w"], H_pre=p["b_pre"], H_post=p["b_post"], H_res=p["b_res"])
    ys, gs = nm.mhc_static_fwd_bwd(x, ps, dy, 20, 1e-6, dtype=torch.float64)
    assert rel_err(yd, ys) < 1e-14
    assert rel_err(gd["x"], gs["x"]) < 1e-13
    assert rel_err(gd["b_res"], gs["H_res"]) < 1e-12
    assert rel_err(gd["b_pre"], gs["H_pre"]) < 1e-12
    assert rel_err(gd["b_post"], gs["H_post"]) < 1e-12


@pytest.mark.parametrize("n,C,T,inject", [(4, 8, 20, False), (8, 8, 4, False), (2, 8, 3, True)])
def test_c_oracle_analytic_backward_against_finite_differences(n, C, T, inject):
    """Central differences of <y, dy> along random directions, fp64."""
    rng = np.random.default_rng(n * 100 + T)
    B, D, eps = 2, n * n + 2 * n, 1e-4
    x = rng.standard_normal((B, n, C)); dy = rng.standard_normal((B, n, C))
    w = 1 + 0.3 * rng.standard_normal(C)
    phi = 0.3 * rng.standard_normal((D, n * C)); bias = 0.4 * rng.standard_normal(D)
    alpha = np.array([0.7, -0.5, 0.9])
    f = rng.standard_normal((B, C)) if inject else None
    g = c_oracle.dynamic_backward(x, dy, w, phi, bias, alpha, T, eps, f)

    def loss(x_=x, w_=w, phi_=phi, bias_=bias, alpha_=alpha, f_=f):
        y, *_ = c_oracle.dynamic_forward(x_, w_, phi_, bias_, alpha_, T, eps, f_)
        return float((y * dy).sum())

    h = 1e-6
    names = [("x", x), ("phi", phi), ("bias", bias), ("alpha", alpha)]
    names.append(("f", f) if inject else ("w", w))
    for name, val in names:
        d = rng.standard_normal(val.shape)
        kw = {name + "_": val + h * d}
        kw2 = {name + "_": val - h * d}
        fd = (loss(**kw) - loss(**kw2)) / (2 * h)
        an = float((g[name] * d).sum())
        assert abs(fd - an) <= 2e-6 * max(1.0, abs(an)), (name, fd, an)


def test_plain_sinkhorn_operator_reference():
    g = torch.Generator().manual_seed(1)
    inp = torch.rand(32, 32, generator=g, dtype=torch.float64) + 0.1
    out = nm.sinkhorn_knopp_plain(inp, 50, 1e-8)
    assert (out.sum(0) - 1).abs().max() < 1e-9 and (out.sum(1) - 1).abs().max() < 1e-6
    z = torch.zeros(4, 4, dtype=torch.float64)
    assert torch.equal(nm.sinkhorn_knopp_plain(z, 3, 1e-8), z)  # thresholded: no 0/0


def test_rmsnorm_backward_reference_is_autograd():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 32, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(32, generator=g, dtype=torch.float64, requires_grad=True)
    go = torch.randn(6, 32, generator=g, dtype=torch.float64)
    nm.rmsnorm(x, w, 1e-5).backward(go)
    dx, dw = nm.rmsnorm_backward_ref(go, x.detach(), w.detach(), 1e-5)
    assert rel_err(dx, x.grad) < 1e-13 and rel_err(dw, w.grad) < 1e-13


def test_plain_sinkhorn_one_iteration_closed_form_on_a_non_square_matrix():
    """One iteration is: rows divided by their sums, THEN columns divided by the sums of that
    result.  On a 2 x 3 matrix worked by hand the two orders give different answers, and a
    transposed operand (columns first) fails; both restatements must give the row-then-column one."""
    a = np.array([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    rows_first = a / a.sum(1, keepdims=True)                  # [[1/6, 1/3, 1/2], [4/15, 1/3, 2/5]]
    want = rows_first / rows_first.sum(0, keepdims=True)
    hand = np.array([[(1 / 6) / (1 / 6 + 4 / 15), 0.5, 0.5 / 0.9], [(4 / 15) / (1 / 6 + 4 / 15), 0.5, 0.4 / 0.9]])
    assert np.allclose(want, hand, rtol=0, atol=1e-15)
    cols_first = a / a.sum(0, keepdims=True)
    cols_first = cols_first / cols_first.sum(1, keepdims=True)
    assert np.abs(cols_first - want).max() > 1e-2             # the two orders are far apart
    got_c = c_oracle.sinkhorn_plain_forward(a, 1, 1e-8)
    got_t = nm.sinkhorn_knopp_plain(torch.from_numpy(a), 1, 1e-8).numpy()
    assert np.abs(got_c - want).max() < 1e-15 and np.abs(got_t - want).max() < 1e-15
    # after a column step every column sums to one exactly; the rows of a 2 x 3 matrix sum to 3/2
    # in the limit (total mass = number of columns), not to one
    far = c_oracle.sinkhorn_plain_forward(a, 200, 1e-8)
    assert np.abs(far.sum(0) - 1).max() < 1e-14 and np.abs(far.sum(1) - 1.5).max() < 1e-12
    # the threshold: a row whose sum does not exceed eps is left alone (no 0/0), the others are not
    z = np.array([[0.0, 0.0, 0.0], [1.0, 1.0, 2.0]])
    out = c_oracle.sinkhorn_plain_forward(z, 1, 1e-8)
    assert np.array_equal(out[0], np.zeros(3)) and np.allclose(out[1], [1.0, 1.0, 1.0])


@pytest.mark.parametrize("rows,cols,T", [(4, 4, 5), (3, 7, 4), (6, 2, 3), (5, 5, 0)])
def test_c_oracle_plain_sinkhorn_matches_torch_and_finite_differences(rows, cols, T):
    rng = np.random.default_rng(rows * 10 + cols)
    inp = rng.random((rows, cols)) + 0.2
    go = rng.standard_normal((rows, cols))
    out_c = c_oracle.sinkhorn_plain_forward(inp, T, 1e-8)
    t = torch.from_numpy(inp).requires_grad_(True)
    out_t = nm.sinkhorn_knopp_plain(t, T, 1e-8)
    assert np.abs(out_c - out_t.detach().numpy()).max() < 1e-14
    out_t.backward(torch.from_numpy(go))
    d_c = c_oracle.sinkhorn_plain_backward(go, inp, T, 1e-8)
    assert np.abs(d_c - t.grad.numpy()).max() < 1e-12 * max(1.0, np.abs(d_c).max())
    d = rng.standard_normal((rows, cols))
    h = 1e-6
    fd = ((c_oracle.sinkhorn_plain_forward(inp + h * d, T, 1e-8) - c_oracle.sinkhorn_plain_forward(inp - h * d, T, 1e-8))
          * go).sum() / (2 * h)
    assert abs(fd - (d_c * d).sum()) <= 1e-7 * max(1.0, abs(fd))


def test_c_oracle_rmsnorm_against_the_library_routine_and_finite_differences():
    rng = np.random.default_rng(5)
    rows, C, eps = 5, 24, 1e-5
    x, w, go = rng.standard_normal((rows, C)), 1 + 0.3 * rng.standard_normal(C), rng.standard_normal((rows, C))
    out, rms = c_oracle.rmsnorm_forward(x, w, eps)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x), (C,), torch.from_numpy(w), eps).numpy()
    assert np.abs(out - ref).max() < 1e-14
    assert np.abs(rms - np.sqrt((x * x).mean(1) + eps)).max() < 1e-15
    d_x, d_w = c_oracle.rmsnorm_backward(go, x, w, rms)
    h = 1e-6
    for name, val, grad in (("x", x, d_x), ("w", w, d_w)):
        d = rng.standard_normal(val.shape)
        f = lambda v: (c_oracle.rmsnorm_forward(v if name == "x" else x, v if name == "w" else w, eps)[0] * go).sum()
        fd = (f(val + h * d) - f(val - h * d)) / (2 * h)
        assert abs(fd - (grad * d).sum()) <= 1e-7 * max(1.0, abs(fd)), name
