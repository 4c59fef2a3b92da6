"""Autograd glue over the HIP library: the operator surface of the reference's mhc.ops
(src/python/mhc/ops.py) with the same names, argument order and dtype contract.

Differences that a caller can observe are limited to these:
* results follow the naive PyTorch layer exactly (eps added to the Sinkhorn denominators,
  exact Sinkhorn backward, per-sample coefficients in the dynamic backward);
* float32 inputs are computed in float32 end to end; bfloat16 inputs stay bfloat16 in HBM
  (fp32 accumulation) instead of being up-cast first;
* no host synchronisation (the alphas are read on the device) and no Python loop over samples.
"""
from __future__ import annotations

import weakref

import torch
from torch.autograd import Function

from . import _lib
from ._lib import check, dtype_code, lib, ptr, require_gpu, stream_ptr, workspace


def _act(x: torch.Tensor) -> torch.Tensor:
    """Activations travel as float32 or bfloat16; anything else is widened like the reference's .float()."""
    return x if x.dtype in (torch.float32, torch.bfloat16) else x.float()


# ----------------------------------------------------------------------------------------------
# stand-alone operators (reference ops.py:13-52)
# ----------------------------------------------------------------------------------------------
class SinkhornKnoppFunction(Function):
    @staticmethod
    def forward(ctx, inp, num_iters, eps):
        inp = inp.contiguous()
        require_gpu(inp)
        rows, cols = inp.shape[-2], inp.shape[-1]
        batch = inp.numel() // (rows * cols)
        out = torch.empty_like(inp)
        check("mhc_sinkhorn_knopp_fwd",
              lib.mhc_sinkhorn_knopp_fwd(ptr(inp), ptr(out), batch, rows, cols, int(num_iters),
                                         float(eps), stream_ptr(inp.device)))
        ctx.save_for_backward(inp)
        ctx.num_iters, ctx.eps = int(num_iters), float(eps)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        (inp,) = ctx.saved_tensors
        grad_output = grad_output.contiguous().float()
        rows, cols = inp.shape[-2], inp.shape[-1]
        batch = inp.numel() // (rows * cols)
        d_inp = torch.empty_like(inp)
        nbytes = lib.mhc_sinkhorn_knopp_bwd_workspace_bytes(batch, rows, cols, ctx.num_iters)
        ws = workspace(inp.device, nbytes)
        check("mhc_sinkhorn_knopp_bwd",
              lib.mhc_sinkhorn_knopp_bwd(ptr(grad_output), ptr(inp), ptr(d_inp), batch, rows, cols,
                                         ctx.num_iters, ctx.eps, ptr(ws), ws.numel(),
                                         stream_ptr(inp.device)))
        return d_inp, None, None


class RMSNormFunction(Function):
    @staticmethod
    def forward(ctx, inp, weight, eps):
        inp, weight = inp.contiguous(), weight.contiguous()
        require_gpu(inp, weight)
        C = inp.shape[-1]
        rows = inp.numel() // C
        out = torch.empty_like(inp)
        rms = torch.empty(rows, dtype=torch.float32, device=inp.device)
        check("mhc_rmsnorm_fwd",
              lib.mhc_rmsnorm_fwd(ptr(inp), dtype_code(inp), ptr(weight), dtype_code(weight), ptr(out),
                                  ptr(rms), rows, C, float(eps), stream_ptr(inp.device)))
        ctx.save_for_backward(inp, weight, rms)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        inp, weight, rms = ctx.saved_tensors
        grad_output = grad_output.contiguous().to(inp.dtype)
        C = inp.shape[-1]
        rows = inp.numel() // C
        d_inp = torch.empty_like(inp)
        d_w = torch.empty(C, dtype=torch.float32, device=inp.device)
        ws = workspace(inp.device, lib.mhc_rmsnorm_bwd_workspace_bytes(rows, C))
        check("mhc_rmsnorm_bwd",
              lib.mhc_rmsnorm_bwd(ptr(grad_output), ptr(inp), dtype_code(inp), ptr(weight),
                                  dtype_code(weight), ptr(rms), ptr(d_inp), ptr(d_w), rows, C, ptr(ws),
                                  ws.numel(), stream_ptr(inp.device)))
        return d_inp, d_w.to(weight.dtype), None


def sinkhorn_knopp(inp, num_iters=20, eps=1e-8):
    return SinkhornKnoppFunction.apply(inp.float(), num_iters, eps)


def rmsnorm(inp, weight, eps=1e-5):
    return RMSNormFunction.apply(inp.bfloat16(), weight.bfloat16(), eps)


# ----------------------------------------------------------------------------------------------
# static-H layer (reference ops.py:55-151)
# ----------------------------------------------------------------------------------------------
def _w_arg(w):
    return (ptr(w), dtype_code(w)) if w is not None else (None, 0)


class MHCLayerFunction(Function):
    @staticmethod
    def forward(ctx, x_expanded, rmsnorm_weight, H_pre, H_post, H_res, sinkhorn_iters, eps,
                out_dtype=None, f_inject=None):
        x = x_expanded.contiguous()
        w = None if rmsnorm_weight is None else rmsnorm_weight.contiguous()
        H_pre, H_post, H_res = H_pre.contiguous(), H_post.contiguous(), H_res.contiguous()
        f_inject = None if f_inject is None else f_inject.contiguous().to(x.dtype)
        require_gpu(x, w, H_pre, H_post, H_res, f_inject)
        B, n, C = x.shape
        dev = x.device
        y = torch.empty((B, n, C), dtype=out_dtype or torch.float32, device=dev)
        Hp = torch.empty(n, dtype=torch.float32, device=dev)
        Ho = torch.empty(n, dtype=torch.float32, device=dev)
        M = torch.empty((n, n), dtype=torch.float32, device=dev)
        q = torch.empty(B, dtype=torch.float32, device=dev)
        ws = workspace(dev, lib.mhc_layer_static_workspace_bytes(B, n, C))
        wp, wd = _w_arg(w)
        check("mhc_layer_fwd",
              lib.mhc_layer_fwd(ptr(x), dtype_code(x), wp, wd, ptr(H_pre), ptr(H_post), ptr(H_res),
                                ptr(f_inject), ptr(y), dtype_code(y), ptr(Hp), ptr(Ho), ptr(M), ptr(q),
                                B, n, C, int(sinkhorn_iters), float(eps), ptr(ws), ws.numel(),
                                stream_ptr(dev)))
        ctx.save_for_backward(x, w, H_pre, H_post, H_res, f_inject, Hp, Ho, M, q)
        ctx.sinkhorn_iters, ctx.eps = int(sinkhorn_iters), float(eps)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, w, H_pre, H_post, H_res, f_inject, Hp, Ho, M, q = ctx.saved_tensors
        dy = grad_output.contiguous()
        B, n, C = x.shape
        dev = x.device
        dx = torch.empty_like(x)
        df = None if f_inject is None else torch.empty_like(f_inject)
        dw = None if f_inject is not None else torch.empty(C, dtype=torch.float32, device=dev)
        dHp = torch.empty(n, dtype=torch.float32, device=dev)
        dHo = torch.empty(n, dtype=torch.float32, device=dev)
        dHr = torch.empty((n, n), dtype=torch.float32, device=dev)
        ws = workspace(dev, lib.mhc_layer_static_workspace_bytes(B, n, C))
        wp, wd = _w_arg(w)
        check("mhc_layer_bwd",
              lib.mhc_layer_bwd(ptr(dy), dtype_code(dy), ptr(x), dtype_code(x), wp, wd, ptr(H_pre),
                                ptr(H_post), ptr(H_res), ptr(f_inject), ptr(Hp), ptr(Ho), ptr(M), ptr(q),
                                ptr(dx), ptr(df), ptr(dw), ptr(dHp), ptr(dHo), ptr(dHr), B, n, C,
                                ctx.sinkhorn_iters, ctx.eps, ptr(ws), ws.numel(), stream_ptr(dev)))
        dw_out = None if (dw is None or w is None) else dw.to(w.dtype)
        return dx, dw_out, dHp, dHo, dHr, None, None, None, df


def mhc_layer_fused(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, sinkhorn_iters=20, eps=1e-5,
                    out_dtype=None, f_inject=None):
    return MHCLayerFunction.apply(_act(x_expanded), rmsnorm_weight, H_pre.float(), H_post.float(),
                                  H_res.float(), sinkhorn_iters, eps, out_dtype, f_inject)


def mhc_layer_fused_inference(x_expanded, rmsnorm_weight, H_pre, H_post, H_res, sinkhorn_iters=20,
                              eps=1e-5, out_dtype=None):
    """Forward only: no tensors are kept for a backward pass (coefficients stay in the workspace)."""
    x = _act(x_expanded).contiguous()
    w = rmsnorm_weight.contiguous()
    H_pre, H_post, H_res = (t.float().contiguous() for t in (H_pre, H_post, H_res))
    require_gpu(x, w, H_pre, H_post, H_res)
    B, n, C = x.shape
    y = torch.empty((B, n, C), dtype=out_dtype or torch.float32, device=x.device)
    ws = workspace(x.device, lib.mhc_layer_static_workspace_bytes(B, n, C))
    check("mhc_layer_fwd",
          lib.mhc_layer_fwd(ptr(x), dtype_code(x), ptr(w), dtype_code(w), ptr(H_pre), ptr(H_post),
                            ptr(H_res), None, ptr(y), dtype_code(y), None, None, None, None, B, n, C,
                            int(sinkhorn_iters), float(eps), ptr(ws), ws.numel(), stream_ptr(x.device)))
    return y


# ----------------------------------------------------------------------------------------------
# dynamic-H layer (reference ops.py:154-417)
# ----------------------------------------------------------------------------------------------
class _DerivedCache:
    """Small tensors derived from parameters (concatenations, casts), rebuilt only when a source
    changed.  An entry is valid while the very same tensor objects are alive (weak references: a new
    tensor that happens to reuse the address of a freed one never matches) and their storage address
    and in-place version counters are unchanged; it is dropped when one of them is freed."""

    def __init__(self, limit):
        self._d = {}
        self._limit = limit

    def get(self, sources, extra, build):
        key = tuple(id(t) for t in sources) + (extra,)
        state = tuple((t.data_ptr(), t._version, tuple(t.shape)) for t in sources)
        hit = self._d.get(key)
        if hit is not None and hit[0] == state and all(r() is t for r, t in zip(hit[1], sources)):
            return hit[2]
        with torch.no_grad():
            value = build()
        if len(self._d) >= self._limit:
            self._d.clear()
        # the entry (and the derived tensor it holds) goes away with the first source that dies
        drop = lambda _ref, d=self._d, k=key: d.pop(k, None)
        self._d[key] = (state, tuple(weakref.ref(t, drop) for t in sources), value)
        return value


_PHI_CACHE = _DerivedCache(64)
_SMALL_CACHE = _DerivedCache(256)


def _phi_concat(phi_pre, phi_post, phi_res, dtype):
    """[D, nC] = rows [pre | post | res] in `dtype`."""
    n = phi_pre.size(0)
    return _PHI_CACHE.get(
        (phi_pre, phi_post, phi_res), dtype,
        lambda: torch.cat([phi_pre, phi_post, phi_res.reshape(n * n, -1)], dim=0).to(dtype).contiguous())


def _bias_alpha(b_pre, b_post, b_res, alpha_pre, alpha_post, alpha_res, dev):
    """fp32 [D] bias (pre | post | res) and fp32 [3] alpha on the device (two small kernels and
    their launch overhead on every call otherwise)."""
    def build():
        bias = torch.cat([b_pre.reshape(-1), b_post.reshape(-1), b_res.reshape(-1)]).float().to(dev)
        alpha = torch.stack([a.to(dev).reshape(()).float() for a in (alpha_pre, alpha_post, alpha_res)])
        return bias, alpha
    return _SMALL_CACHE.get((b_pre, b_post, b_res, alpha_pre, alpha_post, alpha_res), str(dev), build)


class MHCLayerDynamicFunction(Function):
    @staticmethod
    def forward(ctx, x_expanded, rmsnorm_weight, phi_pre, phi_post, phi_res, alpha_pre, alpha_post,
                alpha_res, b_pre, b_post, b_res, sinkhorn_iters, eps, out_dtype=None, f_inject=None):
        x = x_expanded.contiguous()
        w = None if rmsnorm_weight is None else rmsnorm_weight.contiguous()
        f_inject = None if f_inject is None else f_inject.contiguous().to(x.dtype)
        B, n, C = x.shape
        dev = x.device
        D = n * n + 2 * n
        phi = _phi_concat(phi_pre, phi_post, phi_res,
                          torch.bfloat16 if x.dtype == torch.bfloat16 else torch.float32)
        alphas = tuple(a if torch.is_tensor(a) else torch.as_tensor(a, device=dev)
                       for a in (alpha_pre, alpha_post, alpha_res))
        bias, alpha = _bias_alpha(b_pre, b_post, b_res, *alphas, dev)
        require_gpu(x, w, phi, bias, alpha, f_inject)
        f32 = dict(dtype=torch.float32, device=dev)
        y = torch.empty((B, n, C), dtype=out_dtype or torch.float32, device=dev)
        Hp, Ho = torch.empty((B, n), **f32), torch.empty((B, n), **f32)
        M, P = torch.empty((B, n, n), **f32), torch.empty((B, D), **f32)
        r, q = torch.empty(B, **f32), torch.empty(B, **f32)
        ws = workspace(dev, lib.mhc_layer_dynamic_workspace_bytes(B, n, C))
        wp, wd = _w_arg(w)
        check("mhc_layer_fwd_dynamic",
              lib.mhc_layer_fwd_dynamic(ptr(x), dtype_code(x), wp, wd, ptr(phi), dtype_code(phi),
                                        ptr(bias), ptr(alpha), ptr(f_inject), ptr(y), dtype_code(y),
                                        ptr(Hp), ptr(Ho), ptr(M), ptr(P), ptr(r), ptr(q), B, n, C,
                                        int(sinkhorn_iters), float(eps), ptr(ws), ws.numel(),
                                        stream_ptr(dev)))
        ctx.save_for_backward(x, w, phi, bias, alpha, f_inject, Hp, Ho, M, P, r, q)
        ctx.sinkhorn_iters, ctx.eps = int(sinkhorn_iters), float(eps)
        ctx.param_dtypes = (phi_pre.dtype, phi_post.dtype, phi_res.dtype,
                            *(torch.as_tensor(a).dtype for a in (alpha_pre, alpha_post, alpha_res)),
                            b_pre.dtype, b_post.dtype, b_res.dtype)
        ctx.b_res_shape = tuple(b_res.shape)
        ctx.alpha_is_tensor = tuple(torch.is_tensor(a) for a in (alpha_pre, alpha_post, alpha_res))
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, w, phi, bias, alpha, f_inject, Hp, Ho, M, P, r, q = ctx.saved_tensors
        dy = grad_output.contiguous()
        B, n, C = x.shape
        dev = x.device
        D = n * n + 2 * n
        f32 = dict(dtype=torch.float32, device=dev)
        dx = torch.empty_like(x)
        df = None if f_inject is None else torch.empty_like(f_inject)
        dw = None if f_inject is not None else torch.empty(C, **f32)
        dphi = torch.empty((D, n * C), **f32)
        dbias, dalpha = torch.empty(D, **f32), torch.empty(3, **f32)
        ws = workspace(dev, lib.mhc_layer_dynamic_workspace_bytes(B, n, C))
        wp, wd = _w_arg(w)
        check("mhc_layer_bwd_dynamic",
              lib.mhc_layer_bwd_dynamic(ptr(dy), dtype_code(dy), ptr(x), dtype_code(x), wp, wd, ptr(phi),
                                        dtype_code(phi), ptr(bias), ptr(alpha), ptr(f_inject), ptr(Hp),
                                        ptr(Ho), ptr(M), ptr(P), ptr(r), ptr(q), ptr(dx), ptr(df),
                                        ptr(dw), ptr(dphi), ptr(dbias), ptr(dalpha), B, n, C,
                                        ctx.sinkhorn_iters, ctx.eps, ptr(ws), ws.numel(),
                                        stream_ptr(dev)))
        dt = ctx.param_dtypes
        ait = ctx.alpha_is_tensor
        dw_out = None if (dw is None or w is None) else dw.to(w.dtype)
        return (dx, dw_out,
                dphi[:n].to(dt[0]), dphi[n:2 * n].to(dt[1]), dphi[2 * n:].to(dt[2]),
                dalpha[0].to(dt[3]) if ait[0] else None,
                dalpha[1].to(dt[4]) if ait[1] else None,
                dalpha[2].to(dt[5]) if ait[2] else None,
                dbias[:n].to(dt[6]), dbias[n:2 * n].to(dt[7]),
                dbias[2 * n:].reshape(ctx.b_res_shape).to(dt[8]),
                None, None, None, df)


def mhc_layer_fused_dynamic(x_expanded, rmsnorm_weight, phi_pre, phi_post, phi_res, alpha_pre,
                            alpha_post, alpha_res, b_pre, b_post, b_res, sinkhorn_iters=20, eps=1e-5,
                            out_dtype=None, f_inject=None):
    dev = phi_pre.device
    if not torch.is_tensor(alpha_pre):
        alpha_pre = torch.tensor(alpha_pre, device=dev, dtype=phi_pre.dtype)
    if not torch.is_tensor(alpha_post):
        alpha_post = torch.tensor(alpha_post, device=dev, dtype=phi_pre.dtype)
    if not torch.is_tensor(alpha_res):
        alpha_res = torch.tensor(alpha_res, device=dev, dtype=phi_pre.dtype)
    return MHCLayerDynamicFunction.apply(_act(x_expanded), rmsnorm_weight, phi_pre, phi_post, phi_res,
                                         alpha_pre, alpha_post, alpha_res, b_pre, b_post, b_res,
                                         sinkhorn_iters, eps, out_dtype, f_inject)
