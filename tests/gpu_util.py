"""Runs the HIP path (through the mhc package, i.e. through the C ABI) on tensors given on the
CPU and returns results on the CPU under the oracle's names."""
import torch

from oracle import naive_mhc as nm


def _dev(t, dtype=None):
    t = torch.as_tensor(t)
    if dtype is not None:
        t = t.to(dtype)
    return t.detach().to("cuda").contiguous()


def hip_dynamic(x, params, dy, T, eps, f_inject=None, act_dtype=torch.float32, out_dtype=None,
                w_dtype=torch.float32):
    """Forward + backward of mhc.mhc_layer_fused_dynamic.  Returns (y, grads) like
    oracle.naive_mhc.mhc_dynamic_fwd_bwd."""
    import mhc

    xd = _dev(x, act_dtype).requires_grad_(True)
    p = {}
    for k in nm.DYN_PARAM_NAMES:
        dt = w_dtype if k == "w" else torch.float32
        p[k] = _dev(params[k], dt).requires_grad_(True)
    fd = None if f_inject is None else _dev(f_inject, act_dtype).requires_grad_(True)
    y = mhc.mhc_layer_fused_dynamic(xd, p["w"], p["phi_pre"], p["phi_post"], p["phi_res"],
                                    p["alpha_pre"], p["alpha_post"], p["alpha_res"], p["b_pre"],
                                    p["b_post"], p["b_res"], T, eps, out_dtype, fd)
    y.backward(_dev(dy, y.dtype))
    torch.cuda.synchronize()
    grads = {"x": xd.grad.float().cpu()}
    for k in nm.DYN_PARAM_NAMES:
        if p[k].grad is not None:
            grads[k] = p[k].grad.float().cpu()
    if fd is not None:
        grads["f"] = fd.grad.float().cpu()
    return y.detach().float().cpu(), grads


def hip_static(x, params, dy, T, eps, f_inject=None, act_dtype=torch.float32, out_dtype=None,
               w_dtype=torch.float32):
    import mhc

    xd = _dev(x, act_dtype).requires_grad_(True)
    p = {}
    for k in nm.STATIC_PARAM_NAMES:
        dt = w_dtype if k == "w" else torch.float32
        p[k] = _dev(params[k], dt).requires_grad_(True)
    fd = None if f_inject is None else _dev(f_inject, act_dtype).requires_grad_(True)
    y = mhc.mhc_layer_fused(xd, p["w"], p["H_pre"], p["H_post"], p["H_res"], T, eps, out_dtype, fd)
    y.backward(_dev(dy, y.dtype))
    torch.cuda.synchronize()
    grads = {"x": xd.grad.float().cpu()}
    for k in nm.STATIC_PARAM_NAMES:
        if p[k].grad is not None:
            grads[k] = p[k].grad.float().cpu()
    if fd is not None:
        grads["f"] = fd.grad.float().cpu()
    return y.detach().float().cpu(), grads
