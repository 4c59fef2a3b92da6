"""Operator surface of the reference's mhc.ops (src/python/mhc/ops.py): same names, argument order
and dtype contract, served by the PyTorch-ROCm extension mhc_torch_ext (C++: output allocation,
current-stream lookup and the autograd functions) over the C ABI of libmhc_hip.so.

Differences that a caller can observe are limited to these:
* results follow the naive PyTorch layer exactly (eps added to the Sinkhorn denominators,
  exact Sinkhorn backward, per-sample coefficients in the dynamic backward);
* float32 inputs are computed in float32 end to end; bfloat16 inputs stay bfloat16 in HBM
  (fp32 accumulation) instead of being up-cast first;
* no host synchronisation (the alphas are read on the device) and no Python loop over samples.

The dynamic layer gathers its parameters (three phi matrices, biases, alphas) into the library's
layout with one small launch per forward call, as the reference re-concatenates them on every call
(ops.py:172-177).  `set_param_cache(True)` reuses the gathered copy while the parameters' storage
addresses and in-place version counters are unchanged; writes through `.data` do not bump those
counters, so the cache is off unless asked for.
"""
from __future__ import annotations

import torch

from . import _lib

try:
    from . import mhc_torch_ext as _ext
except ImportError as exc:  # no fallback: the operators need the compiled extension
    raise ImportError(
        "mhc_torch_ext (the PyTorch-ROCm extension) is not built. Build it first:\n"
        "    python mhc.cu_amd/build.py") from exc

if _ext.abi_version() != _lib.ABI_VERSION:
    raise ImportError(f"mhc_torch_ext was built against ABI {_ext.abi_version()}, binding expects {_lib.ABI_VERSION}")
_ext.set_error_class(_lib.MHCError)


def set_param_cache(enabled: bool) -> None:
    """Opt in to (or out of) reusing the gathered phi / bias / alpha of a dynamic layer between calls."""
    _ext.set_param_cache(bool(enabled))


# ----------------------------------------------------------------------------------------------
# stand-alone operators (reference ops.py:13-52)
# ----------------------------------------------------------------------------------------------
class SinkhornKnoppFunction:
    """Autograd function of mhc.sinkhorn_knopp (implemented in the extension); `apply` as on a
    torch.autograd.Function."""

    @staticmethod
    def apply(inp, num_iters, eps):
        return _ext.sinkhorn_knopp(inp, int(num_iters), float(eps))


class RMSNormFunction:
    @staticmethod
    def apply(inp, weight, eps):
        return _ext.rmsnorm(inp, weight, float(eps))


def sinkhorn_knopp(inp, num_iters=20, eps=1e-8):
    """Sinkhorn-Knopp normalisation of a [rows, cols] or [batch, rows, cols] matrix with an exact
    backward (reference ops.py:13-32).  Limits of the HIP operator: rows, cols <= 128 and
    num_iters <= 1024; beyond them the call raises MHCError (bad shape)."""
    return _ext.sinkhorn_knopp(inp.float(), int(num_iters), float(eps))


def rmsnorm(inp, weight, eps=1e-5):
    """RMSNorm over the last dimension in bfloat16 with float32 accumulation (reference
    ops.py:35-52); any number of rows, row length limited by device memory only."""
    return _ext.rmsnorm(inp.bfloat16(), weight.bfloat16(), float(eps))


# ----------------------------------------------------------------------------------------------
# static-H layer (reference ops.py:55-151)
# ----------------------------------------------------------------------------------------------
class MHCLayerFunction:
    @staticmethod
    def apply(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, sinkhorn_iters, eps, out_dtype=None,
              f_inject=None):
        return _ext.mhc_layer_static(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, int(sinkhorn_iters),
                                     float(eps), out_dtype, f_inject)


def mhc_layer_fused(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, sinkhorn_iters=20, eps=1e-5,
                    out_dtype=None, f_inject=None):
    return _ext.mhc_layer_static(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, int(sinkhorn_iters),
                                 float(eps), out_dtype, f_inject)


def mhc_layer_fused_inference(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, sinkhorn_iters=20,
                              eps=1e-5, out_dtype=None):
    """Forward only: no tensors are kept for a backward pass (coefficients stay in the workspace)."""
    return _ext.mhc_layer_inference(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, int(sinkhorn_iters),
                                    float(eps), out_dtype)


# ----------------------------------------------------------------------------------------------
# dynamic-H layer (reference ops.py:154-417)
# ----------------------------------------------------------------------------------------------
def _as_tensor(a, like):
    return a if torch.is_tensor(a) else torch.tensor(a, device=like.device, dtype=like.dtype)


class MHCLayerDynamicFunction:
    @staticmethod
    def apply(x_expanded, rmsnorm_weight, phi_pre, phi_post, phi_res, alpha_pre, alpha_post, alpha_res,
              b_pre, b_post, b_res, sinkhorn_iters, eps, out_dtype=None, f_inject=None):
        return mhc_layer_fused_dynamic(x_expanded, rmsnorm_weight, phi_pre, phi_post, phi_res, alpha_pre,
                                       alpha_post, alpha_res, b_pre, b_post, b_res, sinkhorn_iters, eps,
                                       out_dtype, f_inject)


def mhc_layer_fused_dynamic(x_expanded, rmsnorm_weight, phi_pre, phi_post, phi_res, alpha_pre,
                            alpha_post, alpha_res, b_pre, b_post, b_res, sinkhorn_iters=20, eps=1e-5,
                            out_dtype=None, f_inject=None, compute_bf16=False):
    """compute_bf16: float32 activations go through the bf16 (matrix-core) kernels, as in the reference's
    fused path (bindings.cu:421-423); where the kernels load float32 storage themselves no cast pass
    is launched."""
    return _ext.mhc_layer_dynamic(x_expanded, rmsnorm_weight, phi_pre, phi_post, phi_res,
                                  _as_tensor(alpha_pre, phi_pre), _as_tensor(alpha_post, phi_pre),
                                  _as_tensor(alpha_res, phi_pre), b_pre, b_post, b_res, int(sinkhorn_iters),
                                  float(eps), out_dtype, f_inject, bool(compute_bf16))
