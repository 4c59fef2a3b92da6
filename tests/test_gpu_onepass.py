"""The one-launch dynamic forward (projection + coefficients + mix, samples resident in LDS)
through the C ABI: against the oracle at the bf16 tolerance, and against the two-launch path of the
same library on the same inputs (both accumulate bf16 products in fp32, so their saved fp32
tensors agree far inside the bf16 bar).  The group size G (samples per workgroup) is forced through
the library's experiment hook so that ragged last groups and G > 8 (two row pieces per lane) are
covered at small sizes."""
import pytest
import torch

from helpers import rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu

K_OFF, K_G = 0, 1


def _tune(key, value):
    from mhc._lib import tuning_lib

    assert tuning_lib().mhc_tuning_set(key, value) == 0


@pytest.fixture(autouse=True)
def _reset_tuning():
    yield
    for k in (K_OFF, K_G):
        _tune(k, 0)


def _forward(B, n, C, x, w, phi, bias, alpha, f, out_dtype, T, eps):
    from mhc import _lib
    from mhc._lib import check, dtype_code, ptr

    lib = _lib.tuning_lib()  # the build of the library whose launch heuristics can be overridden

    D = n * n + 2 * n
    f32 = dict(dtype=torch.float32, device="cuda")
    out = dict(y=torch.empty(B, n, C, dtype=out_dtype, device="cuda"), Hp=torch.empty(B, n, **f32),
               Ho=torch.empty(B, n, **f32), M=torch.empty(B, n, n, **f32), P=torch.empty(B, D, **f32),
               r=torch.empty(B, **f32), q=torch.empty(B, **f32),
               sk=torch.empty(lib.mhc_layer_sinkhorn_state_floats(B, n, T), **f32))
    for t in out.values():
        t.fill_(float("nan"))
    ws = torch.empty(lib.mhc_layer_dynamic_workspace_bytes(B, n, C), dtype=torch.uint8, device="cuda")
    check("mhc_layer_fwd_dynamic",
          lib.mhc_layer_fwd_dynamic(ptr(x), dtype_code(x), ptr(w), dtype_code(w), ptr(phi), dtype_code(phi),
                                    ptr(bias), ptr(alpha), ptr(f), ptr(out["y"]), dtype_code(out["y"]),
                                    ptr(out["Hp"]), ptr(out["Ho"]), ptr(out["M"]), ptr(out["P"]), ptr(out["r"]),
                                    ptr(out["q"]), ptr(out["sk"]), B, n, C, T, eps, ptr(ws), ws.numel(), _lib.stream_ptr(x.device)))
    torch.cuda.synchronize()
    return {k: v.float().cpu() for k, v in out.items()}


CASES = [  # B, n, C, G
    (37, 4, 64, 0), (37, 4, 64, 3), (37, 4, 64, 16), (37, 4, 64, 11), (1, 4, 16, 0),
    (9, 2, 32, 4), (13, 3, 64, 5), (21, 4, 1280, 2), (12, 4, 2560, 5), (33, 1, 64, 9),
    (7, 4, 40, 2), (300, 4, 128, 0),
]


@pytest.mark.parametrize("B,n,C,G", CASES)
@pytest.mark.parametrize("inject", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_onepass_forward(B, n, C, G, inject, out_dtype):
    T, eps = 20, 1e-6
    xh, _, fh, p = nm.make_dynamic_inputs(B, n, C, bf16_round=True, with_f=True)
    for k in ("alpha_pre", "alpha_post", "alpha_res"):
        p[k] = torch.tensor(0.5)  # coefficients that really depend on x
    g = torch.Generator().manual_seed(B * 131 + C)
    p["b_pre"], p["b_post"] = 0.3 * torch.randn(n, generator=g), 0.3 * torch.randn(n, generator=g)
    p["b_res"] = 0.3 * torch.randn(n, n, generator=g)
    p["w"] = (1 + 0.1 * torch.randn(C, generator=g)).bfloat16().float()
    fh = fh if inject else None
    y_ref = nm.mhc_dynamic_forward(xh, p["w"], p["phi_pre"], p["phi_post"], p["phi_res"], p["alpha_pre"],
                                   p["alpha_post"], p["alpha_res"], p["b_pre"], p["b_post"], p["b_res"], T, eps,
                                   f_inject=fh)
    dev = lambda t, dt: t.to(dt).cuda().contiguous()
    x, w = dev(xh, torch.bfloat16), dev(p["w"], torch.bfloat16)
    phi = dev(torch.cat([p["phi_pre"], p["phi_post"], p["phi_res"]], 0), torch.bfloat16)
    bias = dev(torch.cat([p["b_pre"], p["b_post"], p["b_res"].reshape(-1)]), torch.float32)
    alpha = dev(torch.stack([p["alpha_pre"], p["alpha_post"], p["alpha_res"]]), torch.float32)
    f = None if fh is None else dev(fh, torch.bfloat16)

    _tune(K_OFF, 1)
    two = _forward(B, n, C, x, w, phi, bias, alpha, f, out_dtype, T, eps)
    _tune(K_OFF, 2)
    _tune(K_G, G)
    one = _forward(B, n, C, x, w, phi, bias, alpha, f, out_dtype, T, eps)

    # rows and columns n..NP-1 of the saved Sinkhorn denominators are padding nobody reads
    NP = one["sk"].numel() // (B * (T + 1) * 2)
    for o in (one, two):
        o["sk"] = o["sk"].reshape(B, T + 1, 2, NP)[:, :T, :, :n]
    for k, v in one.items():
        assert torch.isfinite(v).all(), k
    e = rel_err(one["y"], y_ref)
    assert e <= 2e-2, f"y vs oracle: {e:.3e}"
    bad = (one["y"] - y_ref).abs() > 2e-2 * y_ref.abs() + 1e-2
    assert not bad.any()
    # same arithmetic up to summation order: the fp32 tensors saved for the backward agree closely
    for k in ("Hp", "Ho", "M", "P", "r", "q", "sk"):
        e = rel_err(one[k], two[k])
        assert e <= 2e-5, f"{k} vs two-launch path: {e:.3e}"
    e = rel_err(one["y"], two["y"])
    assert e <= (1e-2 if out_dtype == torch.bfloat16 else 1e-4), f"y vs two-launch path: {e:.3e}"
