"""The oracle (PyTorch restatement and plain-C restatement) against golden vectors that were
written from the reference's own naive layers (tests/golden/make_golden.py).  CPU only."""
import numpy as np
import pytest
import torch

from helpers import golden, rel_err
from oracle import c_oracle, naive_mhc as nm

TOL = 1e-12  # everything is fp64; only summation order differs


def _t(a):
    return torch.from_numpy(np.asarray(a)).double()


@pytest.mark.parametrize("tag", ["n4", "n8"])
def test_static_torch_oracle_matches_reference(tag):
    g = golden("static_" + tag)
    p = {k: _t(g[k]) for k in ("w", "H_pre", "H_post", "H_res")}
    y, grads = nm.mhc_static_fwd_bwd(_t(g["x"]), p, _t(g["dy"]), int(g["T"]), float(g["eps"]),
                                     dtype=torch.float64)
    assert rel_err(y, g["y"]) < TOL
    assert rel_err(grads["x"], g["dx"]) < TOL
    for k in ("w", "H_pre", "H_post", "H_res"):
        assert rel_err(grads[k], g["d" + k]) < TOL, k


@pytest.mark.parametrize("tag", ["n4", "n8", "n3"])
def test_dynamic_torch_oracle_matches_reference_module(tag):
    """NaiveMHCLayerDynamic keeps phi as [nC, n]; the oracle takes MHCLayer's [n, nC]."""
    g = golden("dynamic_" + tag)
    p = {k: _t(g[k]) for k in nm.DYN_PARAM_NAMES}
    for k in ("phi_pre", "phi_post", "phi_res"):
        p[k] = p[k].t().contiguous()
    y, grads = nm.mhc_dynamic_fwd_bwd(_t(g["x"]), p, _t(g["dy"]), int(g["T"]), float(g["eps"]),
                                      dtype=torch.float64)
    assert rel_err(y, g["y"]) < TOL
    assert rel_err(grads["x"], g["dx"]) < TOL
    for k in nm.DYN_PARAM_NAMES:
        ref = g["d" + k].T if k.startswith("phi") else g["d" + k]
        assert rel_err(grads[k], ref) < TOL, k


@pytest.mark.parametrize("tag", ["n4", "n16"])
def test_dynamic_torch_oracle_matches_reference_functional(tag):
    g = golden("functional_" + tag)
    p = {k: _t(g[k]) for k in nm.DYN_PARAM_NAMES}
    y, grads = nm.mhc_dynamic_fwd_bwd(_t(g["x"]), p, _t(g["dy"]), int(g["T"]), float(g["eps"]),
                                      dtype=torch.float64)
    assert rel_err(y, g["y"]) < TOL
    assert rel_err(grads["x"], g["dx"]) < TOL
    for k in nm.DYN_PARAM_NAMES:
        assert rel_err(grads[k], g["d" + k]) < TOL, k


@pytest.mark.parametrize("tag", ["n4", "n16"])
def test_c_oracle_matches_reference_functional(tag):
    g = golden("functional_" + tag)
    n = int(g["n"])
    phi = np.concatenate([g["phi_pre"], g["phi_post"], g["phi_res"]], axis=0)
    bias = np.concatenate([g["b_pre"].ravel(), g["b_post"].ravel(), g["b_res"].ravel()])
    alpha = np.array([g["alpha_pre"], g["alpha_post"], g["alpha_res"]], dtype=np.float64)
    T, eps = int(g["T"]), float(g["eps"])
    y, *_ = c_oracle.dynamic_forward(g["x"], g["w"], phi, bias, alpha, T, eps)
    gr = c_oracle.dynamic_backward(g["x"], g["dy"], g["w"], phi, bias, alpha, T, eps)
    assert rel_err(y, g["y"]) < TOL
    assert rel_err(gr["x"], g["dx"]) < TOL
    assert rel_err(gr["w"], g["dw"]) < TOL
    dphi = np.concatenate([g["dphi_pre"], g["dphi_post"], g["dphi_res"]], axis=0)
    dbias = np.concatenate([g["db_pre"].ravel(), g["db_post"].ravel(), g["db_res"].ravel()])
    dalpha = np.array([g["dalpha_pre"], g["dalpha_post"], g["dalpha_res"]])
    assert rel_err(gr["phi"], dphi) < TOL
    assert rel_err(gr["bias"], dbias) < TOL
    assert rel_err(gr["alpha"], dalpha) < TOL
    assert n in (4, 16)


@pytest.mark.parametrize("tag", ["n4", "n8"])
def test_c_oracle_matches_reference_static(tag):
    g = golden("static_" + tag)
    logits = np.concatenate([g["H_pre"], g["H_post"], g["H_res"].ravel()])
    T, eps = int(g["T"]), float(g["eps"])
    y, *_ = c_oracle.static_forward(g["x"], g["w"], logits, T, eps)
    gr = c_oracle.static_backward(g["x"], g["dy"], g["w"], logits, T, eps)
    assert rel_err(y, g["y"]) < TOL
    assert rel_err(gr["x"], g["dx"]) < TOL
    assert rel_err(gr["w"], g["dw"]) < TOL
    dlog = np.concatenate([g["dH_pre"], g["dH_post"], g["dH_res"].ravel()])
    assert rel_err(gr["logits"], dlog) < TOL
