"""MHC_F32_AS_BF16 through the C ABI: fp32 activations that the kernels round to bf16 as they load
them (dynamic H, n <= 8, rows that the sample-resident backward holds), against the oracle on the rounded
activations at the bf16 tolerance, and against the same entry points fed bf16 storage.  Shapes the
library does not take in this form are refused with MHC_ERR_BAD_DTYPE before any launch."""
import pytest
import torch

from helpers import pack_dynamic_grads, rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu

T, EPS = 20, 1e-6
MHC_F32_AS_BF16, MHC_ERR_BAD_DTYPE = 2, 4


def _run(B, n, C, storage, inject, seed=0):
    """One forward + backward with x, dy (and f) stored as `storage` ("bf16" or "f32_as_bf16")."""
    from mhc import _lib
    from mhc._lib import check, dtype_code, lib, ptr

    xh, dyh, fh, p = nm.make_dynamic_inputs(B, n, C, seed_data=seed, seed_param=seed + 1, with_f=inject)
    g = torch.Generator().manual_seed(seed + 5)
    for k in ("alpha_pre", "alpha_post", "alpha_res"):
        p[k] = torch.tensor(0.3)
    p["b_res"] = 0.3 * torch.randn(n, n, generator=g)
    p["w"] = (1 + 0.2 * torch.randn(C, generator=g)).bfloat16().float()
    for k in ("phi_pre", "phi_post", "phi_res"):
        p[k] = p[k].bfloat16().float()
    f32 = dict(dtype=torch.float32, device="cuda")
    act = torch.bfloat16 if storage == "bf16" else torch.float32
    dev = lambda t, dt: t.to(dt).cuda().contiguous()
    x, dy = dev(xh, act), dev(dyh, act)
    f = None if fh is None else dev(fh, act)
    w = dev(p["w"], torch.bfloat16)
    phi = dev(torch.cat([p["phi_pre"], p["phi_post"], p["phi_res"]], 0), torch.bfloat16)
    bias = dev(torch.cat([p["b_pre"], p["b_post"], p["b_res"].reshape(-1)]), torch.float32)
    alpha = dev(torch.stack([p["alpha_pre"], p["alpha_post"], p["alpha_res"]]), torch.float32)
    D = n * n + 2 * n
    xc = dtype_code(x) if storage == "bf16" else MHC_F32_AS_BF16
    y = torch.full_like(x, float("nan"))
    Hp, Ho, M = torch.empty(B, n, **f32), torch.empty(B, n, **f32), torch.empty(B, n, n, **f32)
    P, r, q = torch.empty(B, D, **f32), torch.empty(B, **f32), torch.empty(B, **f32)
    sk = torch.empty(max(lib.mhc_layer_sinkhorn_state_floats(B, n, T), 1), **f32)
    ws = torch.empty(lib.mhc_layer_dynamic_workspace_bytes(B, n, C), dtype=torch.uint8, device="cuda")
    st = _lib.stream_ptr(x.device)
    s1 = lib.mhc_layer_fwd_dynamic(ptr(x), xc, ptr(w), dtype_code(w), ptr(phi), dtype_code(phi), ptr(bias), ptr(alpha),
                                   ptr(f), ptr(y), dtype_code(y), ptr(Hp), ptr(Ho), ptr(M), ptr(P), ptr(r), ptr(q), ptr(sk),
                                   B, n, C, T, EPS, ptr(ws), ws.numel(), st)
    out = dict(dx=torch.full_like(x, float("nan")), dw=torch.empty(C, **f32), dphi=torch.empty(D, n * C, **f32),
               dbias=torch.empty(D, **f32), dalpha=torch.empty(3, **f32))
    if f is not None:
        out["df"] = torch.full_like(f, float("nan"))
    s2 = lib.mhc_layer_bwd_dynamic(ptr(dy), dtype_code(dy), ptr(x), xc, ptr(w), dtype_code(w), ptr(phi), dtype_code(phi),
                                   ptr(bias), ptr(alpha), ptr(f), ptr(Hp), ptr(Ho), ptr(M), ptr(P), ptr(r), ptr(q), ptr(sk),
                                   ptr(out["dx"]), ptr(out.get("df")), ptr(out["dw"]), ptr(out["dphi"]), ptr(out["dbias"]),
                                   ptr(out["dalpha"]), B, n, C, T, EPS, ptr(ws), ws.numel(), st)
    torch.cuda.synchronize()
    if s1 or s2:
        return (s1, s2), None, None
    out["y"] = y
    if f is not None:
        out.pop("dw")
    host = dict(x=xh.bfloat16().float(), dy=dyh.bfloat16().float(), f=None if fh is None else fh.bfloat16().float(), p=p)
    return (0, 0), {k: v.float().cpu() for k, v in out.items()}, host


SHAPES = [(5, 4, 64), (1, 4, 128), (3, 2, 40), (7, 1, 136), (33, 4, 1288), (320, 4, 1280), (16, 8, 256),
          (3, 6, 72), (9, 8, 1288), (257, 8, 136), (768, 3, 64), (2000, 4, 64), (1100, 4, 1280)]


@pytest.mark.parametrize("B,n,C", SHAPES)
@pytest.mark.parametrize("inject", [False, True])
def test_f32_storage_consumed_as_bf16(B, n, C, inject):
    from mhc._lib import lib

    assert lib.mhc_layer_dynamic_accepts_f32_as_bf16(B, n, C, T) == 1
    st, got, h = _run(B, n, C, "f32_as_bf16", inject)
    assert st == (0, 0), st
    _, ref16, _ = _run(B, n, C, "bf16", inject)
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(h["x"], h["p"], h["dy"], T, EPS, f_inject=h["f"], dtype=torch.float32)
    dphi, dbias, dalpha = pack_dynamic_grads(
        {k: g_ref.get(k, torch.zeros_like(torch.as_tensor(h["p"][k]))) for k in nm.DYN_PARAM_NAMES if k != "w"}, n)
    ref = dict(y=y_ref, dx=g_ref["x"], dphi=dphi, dbias=dbias, dalpha=dalpha)
    if inject:
        ref["df"] = g_ref["f"]
    else:
        ref["dw"] = g_ref["w"]
    for k, r in ref.items():
        assert torch.isfinite(got[k]).all(), k
        if n == 1 and not inject and k in ("dphi", "dbias", "dalpha"):
            continue  # one stream: the pre entries are O(eps), see test_gpu_parity.py
        e = rel_err(got[k], r)
        assert e <= 2e-2, f"{k}: normalised err {e:.3e}"
        bad = (got[k].double() - r.double()).abs() > 2e-2 * r.double().abs() + 1e-2
        assert not bad.any(), f"{k}: {int(bad.sum())} elements outside rtol/atol"
    # against bf16 storage of the same values: the same products, different rounding of the outputs
    for k in ("dphi", "dbias", "dalpha") + (() if inject else ("dw",)):
        assert rel_err(got[k], ref16[k]) <= 2e-3, k
    for k in ("y", "dx"):
        assert rel_err(got[k], ref16[k]) <= 1.6e-2, k


@pytest.mark.parametrize("B,n,C", [(8, 12, 64), (8, 4, 8192), (8, 4, 36)])
def test_shapes_without_an_fp32_storage_path_are_refused(B, n, C):
    from mhc._lib import lib

    assert lib.mhc_layer_dynamic_accepts_f32_as_bf16(B, n, C, T) == 0
    st, got, _ = _run(B, n, C, "f32_as_bf16", False)
    assert st[0] == MHC_ERR_BAD_DTYPE and got is None
