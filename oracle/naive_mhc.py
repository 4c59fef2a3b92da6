"""CPU oracle for the mHC layer: a plain-PyTorch restatement of the reference's naive layers.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this module; it is the
checker that the parity tests, the smoke test and the benchmark's CPU-baseline leg compare the
HIP path against.  It runs on the CPU in fp32 or fp64 and uses nothing but elementwise torch
ops, sums and matmul/einsum.

What each function follows in the reference (paths under the reference tree):

* ``sinkhorn_knopp_exp``  - src/python/benchmarks/bench_layer.py:48-53 (static) and :112-117
  (batched); same loop in src/python/tests/test_layer.py:38-41.  exp, then ``iters`` times
  row-normalise followed by column-normalise, ``eps`` ADDED to each denominator.
* ``rmsnorm``             - bench_layer.py:55-57 / :119-121: ``x / sqrt(mean(x^2)+eps) * w``.
* ``mhc_static_forward``  - NaiveMHCLayer.forward, bench_layer.py:59-71.
* ``mhc_dynamic_forward`` - NaiveMHCLayerDynamic.forward, bench_layer.py:123-145, with the
  projection weights in MHCLayer's own layout ``[n, nC] / [n*n, nC]`` (src/python/mhc/layer.py:44-46),
  i.e. exactly ``_naive_mhc_dynamic`` of src/python/tests/test_layer.py:7-50.
* ``sinkhorn_knopp_plain`` - the stand-alone operator's CPU reference,
  src/csrc/tests/test_sinkhorn_knopp.cu:16-47 (no exp; a row/column is divided by its sum only
  when that sum exceeds eps).
* ``rmsnorm_backward_ref`` - src/csrc/tests/test_rmsnorm_backward.cu:17-39.

``f_inject``: the benchmark configurations also describe a kernel-level view in which the
"layer output" ``f [B, C]`` is an independent input instead of ``RMSNorm(x_agg) * w``
(the reference's kernel takes it as the ``y_norm`` argument, src/csrc/kernels/stream_ops.cuh:409-412).
Passing ``f_inject`` selects that view.

Parity pins for this file (tests/test_oracle_*.py): golden vectors written from the reference's
own naive classes (tests/golden), library routines (torch.nn.functional.rms_norm, bmm),
closed forms (uniform logits, n=1, identity mapping), structural identities
(alpha=0 dynamic == static), and fp64 finite differences for every gradient.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


# --------------------------------------------------------------------------------------------
# building blocks
# --------------------------------------------------------------------------------------------

def sinkhorn_knopp_exp(logits: torch.Tensor, iters: int, eps: float) -> torch.Tensor:
    """SK(exp(logits)) over the last two dims (bench_layer.py:48-53, :112-117)."""
    M = torch.exp(logits)
    for _ in range(iters):
        M = M / (M.sum(dim=-1, keepdim=True) + eps)
        M = M / (M.sum(dim=-2, keepdim=True) + eps)
    return M


def sinkhorn_knopp_plain(inp: torch.Tensor, iters: int, eps: float) -> torch.Tensor:
    """Stand-alone operator semantics (test_sinkhorn_knopp.cu:16-47): no exp, threshold form."""
    M = inp.clone()
    for _ in range(iters):
        rs = M.sum(dim=-1, keepdim=True)
        M = torch.where(rs > eps, M / rs, M)
        cs = M.sum(dim=-2, keepdim=True)
        M = torch.where(cs > eps, M / cs, M)
    return M


def rmsnorm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """bench_layer.py:55-57.  ``w=None`` is the weight-free projection norm (:126-128)."""
    rms = torch.sqrt(torch.mean(x * x, dim=-1, keepdim=True) + eps)
    out = x / rms
    return out if w is None else out * w


def rmsnorm_backward_ref(grad, inp, w, eps):
    """Row-wise RMSNorm backward as written in test_rmsnorm_backward.cu:17-39.

    Returns (d_inp, d_weight); inputs are 2-D ``[N, C]`` / ``[C]``.
    """
    N, C = inp.shape
    rms = torch.sqrt((inp * inp).mean(dim=-1, keepdim=True) + eps)
    inv = 1.0 / rms
    gw = grad * w
    dot = (gw * inp).sum(dim=-1, keepdim=True)
    d_inp = gw * inv - inp * dot * inv * inv * inv / C
    d_w = (grad * inp * inv).sum(dim=0)
    return d_inp, d_w


# --------------------------------------------------------------------------------------------
# full layers
# --------------------------------------------------------------------------------------------

@dataclass
class MHCIntermediates:
    H_pre: torch.Tensor      # [n] or [B, n]   sigmoid
    H_post: torch.Tensor     # [n] or [B, n]   2*sigmoid
    M: torch.Tensor          # [n, n] or [B, n, n]
    x_agg: torch.Tensor      # [B, C]
    f: torch.Tensor          # [B, C]   RMSNorm(x_agg)*w, or the injected f
    P: Optional[torch.Tensor] = None    # [B, D]  x_norm @ phi_concat^T   (dynamic only)
    r: Optional[torch.Tensor] = None    # [B]     sqrt(mean(x_flat^2)+eps) (dynamic only)


def mhc_static_forward(x, w, H_pre, H_post, H_res, iters: int, eps: float,
                       f_inject: Optional[torch.Tensor] = None, return_intermediates=False):
    """NaiveMHCLayer.forward (bench_layer.py:59-71).

    x [B,n,C]; w [C]; H_pre,H_post [n] logits; H_res [n,n] logits.
    """
    B, n, C = x.shape
    Hp = torch.sigmoid(H_pre)
    Ho = 2.0 * torch.sigmoid(H_post)
    M = sinkhorn_knopp_exp(H_res, iters, eps)
    x_agg = torch.einsum("i,bic->bc", Hp, x)
    f = rmsnorm(x_agg, w, eps) if f_inject is None else f_inject
    y = torch.einsum("ij,bjc->bic", M, x) + Ho.view(1, n, 1) * f.view(B, 1, C)
    if return_intermediates:
        return y, MHCIntermediates(Hp, Ho, M, x_agg, f)
    return y


def mhc_dynamic_forward(x, w, phi_pre, phi_post, phi_res, alpha_pre, alpha_post, alpha_res,
                        b_pre, b_post, b_res, iters: int, eps: float,
                        f_inject: Optional[torch.Tensor] = None, return_intermediates=False):
    """NaiveMHCLayerDynamic.forward (bench_layer.py:123-145) in MHCLayer's parameter layout.

    x [B,n,C]; w [C]; phi_pre, phi_post [n, nC]; phi_res [n*n, nC] (row i*n+j is the weight
    of H_res[i, j]); b_pre, b_post [n]; b_res [n, n]; alpha_* scalars (python floats or 0-dim
    tensors).
    """
    B, n, C = x.shape
    x_flat = x.reshape(B, n * C)
    r = torch.sqrt(torch.mean(x_flat * x_flat, dim=-1, keepdim=True) + eps)
    x_norm = x_flat / r

    p_pre = x_norm @ phi_pre.t()
    p_post = x_norm @ phi_post.t()
    p_res = x_norm @ phi_res.t()

    t_pre = alpha_pre * p_pre + b_pre
    t_post = alpha_post * p_post + b_post
    t_res = alpha_res * p_res.reshape(B, n, n) + b_res

    Hp = torch.sigmoid(t_pre)
    Ho = 2.0 * torch.sigmoid(t_post)
    M = sinkhorn_knopp_exp(t_res, iters, eps)

    x_agg = torch.einsum("bi,bic->bc", Hp, x)
    f = rmsnorm(x_agg, w, eps) if f_inject is None else f_inject
    y = torch.einsum("bij,bjc->bic", M, x) + Ho.unsqueeze(-1) * f.unsqueeze(1)
    if return_intermediates:
        P = torch.cat([p_pre, p_post, p_res], dim=1)
        return y, MHCIntermediates(Hp, Ho, M, x_agg, f, P=P, r=r.reshape(B))
    return y


# --------------------------------------------------------------------------------------------
# gradients by autograd (what "the naive reference's backward" means)
# --------------------------------------------------------------------------------------------

DYN_PARAM_NAMES = ("w", "phi_pre", "phi_post", "phi_res", "alpha_pre", "alpha_post",
                   "alpha_res", "b_pre", "b_post", "b_res")
STATIC_PARAM_NAMES = ("w", "H_pre", "H_post", "H_res")


def _leaf(t, dtype):
    return t.detach().to(dtype).clone().requires_grad_(True)


def mhc_dynamic_fwd_bwd(x, params: dict, dy, iters: int, eps: float, f_inject=None,
                        dtype=torch.float32):
    """Forward + autograd backward of the dynamic layer.  Returns (y, grads) where grads maps
    'x', every name in DYN_PARAM_NAMES (minus 'w' when f is injected) and, with an injected f,
    'f' to its gradient."""
    xl = _leaf(x, dtype)
    pl = {k: _leaf(torch.as_tensor(params[k]), dtype) for k in DYN_PARAM_NAMES}
    fl = None if f_inject is None else _leaf(f_inject, dtype)
    y = mhc_dynamic_forward(xl, pl["w"], pl["phi_pre"], pl["phi_post"], pl["phi_res"],
                            pl["alpha_pre"], pl["alpha_post"], pl["alpha_res"],
                            pl["b_pre"], pl["b_post"], pl["b_res"], iters, eps, f_inject=fl)
    y.backward(dy.detach().to(dtype))
    grads = {"x": xl.grad}
    for k in DYN_PARAM_NAMES:
        if pl[k].grad is not None:
            grads[k] = pl[k].grad
    if fl is not None:
        grads["f"] = fl.grad
    return y.detach(), grads


def mhc_static_fwd_bwd(x, params: dict, dy, iters: int, eps: float, f_inject=None,
                       dtype=torch.float32):
    xl = _leaf(x, dtype)
    pl = {k: _leaf(torch.as_tensor(params[k]), dtype) for k in STATIC_PARAM_NAMES}
    fl = None if f_inject is None else _leaf(f_inject, dtype)
    y = mhc_static_forward(xl, pl["w"], pl["H_pre"], pl["H_post"], pl["H_res"], iters, eps,
                           f_inject=fl)
    y.backward(dy.detach().to(dtype))
    grads = {"x": xl.grad}
    for k in STATIC_PARAM_NAMES:
        if pl[k].grad is not None:
            grads[k] = pl[k].grad
    if fl is not None:
        grads["f"] = fl.grad
    return y.detach(), grads


# --------------------------------------------------------------------------------------------
# seeded synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------------------------

def make_dynamic_inputs(B, n, C, seed_data=0, seed_param=1, bf16_round=False, with_f=False,
                        phi_std=0.02, alpha=0.01):
    """x, dy (and f) ~ N(0,1); phi ~ N(0, phi_std^2); b = 0; alpha = 0.01; w = 1.

    With ``bf16_round`` every tensor that the bf16 configuration stores in bf16 (x, dy, f, phi, w)
    is rounded to bf16 and returned as fp32, so the CPU oracle and the GPU see identical values.
    """
    gd = torch.Generator().manual_seed(seed_data)
    gp = torch.Generator().manual_seed(seed_param)
    nC = n * C
    x = torch.randn(B, n, C, generator=gd)
    dy = torch.randn(B, n, C, generator=gd)
    f = torch.randn(B, C, generator=gd) if with_f else None
    params = {
        "w": torch.ones(C),
        "phi_pre": torch.randn(n, nC, generator=gp) * phi_std,
        "phi_post": torch.randn(n, nC, generator=gp) * phi_std,
        "phi_res": torch.randn(n * n, nC, generator=gp) * phi_std,
        "alpha_pre": torch.tensor(alpha),
        "alpha_post": torch.tensor(alpha),
        "alpha_res": torch.tensor(alpha),
        "b_pre": torch.zeros(n),
        "b_post": torch.zeros(n),
        "b_res": torch.zeros(n, n),
    }
    if bf16_round:
        rb = lambda t: t.bfloat16().float()
        x, dy = rb(x), rb(dy)
        f = None if f is None else rb(f)
        for k in ("w", "phi_pre", "phi_post", "phi_res"):
            params[k] = rb(params[k])
    return x, dy, f, params


def make_static_inputs(B, n, C, seed_data=0, seed_param=1, with_f=False):
    """x, dy (and f) ~ N(0,1); logits H_pre, H_post [n], H_res [n,n] ~ N(0,1); w = 1."""
    gd = torch.Generator().manual_seed(seed_data)
    gp = torch.Generator().manual_seed(seed_param)
    x = torch.randn(B, n, C, generator=gd)
    dy = torch.randn(B, n, C, generator=gd)
    f = torch.randn(B, C, generator=gd) if with_f else None
    params = {
        "w": torch.ones(C),
        "H_pre": torch.randn(n, generator=gp),
        "H_post": torch.randn(n, generator=gp),
        "H_res": torch.randn(n, n, generator=gp),
    }
    return x, dy, f, params
