"""Shared helpers for the test-suite (oracle access, packing, error metrics)."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def rel_err(got, ref):
    """Tensor-normalised relative error: max|got-ref| / max|ref| (both as float64)."""
    got = torch.as_tensor(got).detach().double().cpu()
    ref = torch.as_tensor(ref).detach().double().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    denom = max(float(ref.abs().max()), 1e-30)
    return float((got - ref).abs().max()) / denom


def pack_dynamic(p):
    """(phi_concat [D,nC], bias [D], alpha [3]) from a dict in MHCLayer layout."""
    phi = torch.cat([torch.as_tensor(p["phi_pre"]), torch.as_tensor(p["phi_post"]),
                     torch.as_tensor(p["phi_res"])], dim=0)
    bias = torch.cat([torch.as_tensor(p["b_pre"]).reshape(-1), torch.as_tensor(p["b_post"]).reshape(-1),
                      torch.as_tensor(p["b_res"]).reshape(-1)])
    alpha = torch.stack([torch.as_tensor(p["alpha_pre"]).reshape(()),
                         torch.as_tensor(p["alpha_post"]).reshape(()),
                         torch.as_tensor(p["alpha_res"]).reshape(())])
    return phi, bias, alpha


def pack_dynamic_grads(g, n):
    """Same packing for a gradient dict (missing entries are zero gradients)."""
    z = lambda k, ref: g[k] if k in g else torch.zeros_like(ref)
    dphi = torch.cat([g["phi_pre"], g["phi_post"], g["phi_res"]], dim=0)
    dbias = torch.cat([g["b_pre"].reshape(-1), g["b_post"].reshape(-1), g["b_res"].reshape(-1)])
    dalpha = torch.stack([g["alpha_pre"].reshape(()), g["alpha_post"].reshape(()),
                          g["alpha_res"].reshape(())])
    return dphi, dbias, dalpha
