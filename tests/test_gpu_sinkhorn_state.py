"""The optional Sinkhorn state of the dynamic calls (row and column denominators of every
iteration, written by mhc_layer_fwd_dynamic, read by mhc_layer_bwd_dynamic) through the C ABI.

The backward from the saved state and the backward that recomputes the iterations (state NULL)
run the same reverse sweep on the same denominators, so their gradients must agree far inside the
fp32 bar; the state itself is checked against the oracle's denominators."""
import pytest
import torch

from helpers import rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu


def _fwd_bwd(B, n, C, dtype, T, eps, seed, with_state):
    from mhc import _lib
    from mhc._lib import check, dtype_code, lib, ptr

    xh, dyh, _, p = nm.make_dynamic_inputs(B, n, C, seed_data=seed, seed_param=seed + 1,
                                           bf16_round=dtype == torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 17)
    for k in ("alpha_pre", "alpha_post", "alpha_res"):
        p[k] = torch.tensor(0.5)  # coefficients that depend on x
    p["b_res"] = 0.5 * torch.randn(n, n, generator=g)
    dev = lambda t, dt: t.to(dt).cuda().contiguous()
    x, dy, w = dev(xh, dtype), dev(dyh, dtype), dev(p["w"], dtype)
    phi = dev(torch.cat([p["phi_pre"], p["phi_post"], p["phi_res"]], 0), dtype)
    bias = dev(torch.cat([p["b_pre"], p["b_post"], p["b_res"].reshape(-1)]), torch.float32)
    alpha = dev(torch.stack([p["alpha_pre"], p["alpha_post"], p["alpha_res"]]), torch.float32)
    D = n * n + 2 * n
    f32 = dict(dtype=torch.float32, device="cuda")
    y = torch.empty_like(x)
    Hp, Ho, M = torch.empty(B, n, **f32), torch.empty(B, n, **f32), torch.empty(B, n, n, **f32)
    P, r, q = torch.empty(B, D, **f32), torch.empty(B, **f32), torch.empty(B, **f32)
    sk = torch.full((max(lib.mhc_layer_sinkhorn_state_floats(B, n, T), 1),), float("nan"), **f32)
    ws = torch.empty(lib.mhc_layer_dynamic_workspace_bytes(B, n, C), dtype=torch.uint8, device="cuda")
    st = _lib.stream_ptr(x.device)
    check("mhc_layer_fwd_dynamic",
          lib.mhc_layer_fwd_dynamic(ptr(x), dtype_code(x), ptr(w), dtype_code(w), ptr(phi), dtype_code(phi), ptr(bias),
                                    ptr(alpha), None, ptr(y), dtype_code(y), ptr(Hp), ptr(Ho), ptr(M), ptr(P), ptr(r),
                                    ptr(q), ptr(sk) if with_state else None, B, n, C, T, eps, ptr(ws), ws.numel(), st))
    out = dict(dx=torch.empty_like(x), dw=torch.empty(C, **f32), dphi=torch.empty(D, n * C, **f32),
               dbias=torch.empty(D, **f32), dalpha=torch.empty(3, **f32))
    check("mhc_layer_bwd_dynamic",
          lib.mhc_layer_bwd_dynamic(ptr(dy), dtype_code(dy), ptr(x), dtype_code(x), ptr(w), dtype_code(w), ptr(phi),
                                    dtype_code(phi), ptr(bias), ptr(alpha), None, ptr(Hp), ptr(Ho), ptr(M), ptr(P),
                                    ptr(r), ptr(q), ptr(sk) if with_state else None, ptr(out["dx"]), None,
                                    ptr(out["dw"]), ptr(out["dphi"]), ptr(out["dbias"]), ptr(out["dalpha"]), B, n, C, T,
                                    eps, ptr(ws), ws.numel(), st))
    torch.cuda.synchronize()
    out = {k: v.float().cpu() for k, v in out.items()}
    out["M"], out["y"] = M.cpu(), y.float().cpu()
    if with_state and T > 0:
        NP = sk.numel() // (B * (T + 1) * 2)
        out["sk"] = sk.reshape(B, T + 1, 2, NP)[:, :T, :, :n].cpu()
        out["P"] = P.cpu()  # rows of RMSNorm(x_flat) @ phi^T: the logits are alpha * P + b
        out["b_res"], out["alpha_res"] = p["b_res"], float(p["alpha_res"])
    return out


CASES = [(5, 1, 64, 20), (9, 3, 48, 20), (33, 4, 128, 20), (7, 4, 64, 1), (6, 4, 64, 0), (11, 6, 64, 20),
         (10, 8, 96, 7), (4, 12, 64, 20), (5, 16, 32, 20), (3, 24, 32, 5), (3, 32, 64, 20)]


@pytest.mark.parametrize("B,n,C,T", CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_from_saved_state_matches_recompute(B, n, C, T, dtype):
    eps = 1e-6
    a = _fwd_bwd(B, n, C, dtype, T, eps, seed=3 * n + B, with_state=True)
    b = _fwd_bwd(B, n, C, dtype, T, eps, seed=3 * n + B, with_state=False)
    for k in ("y", "M"):
        # the forward runs the same arithmetic whether or not the caller keeps the state
        assert torch.equal(a[k], b[k]), (k, rel_err(a[k], b[k]))
    for k in ("dx", "dw", "dphi", "dbias", "dalpha"):
        assert torch.isfinite(a[k]).all(), k
        e = rel_err(a[k], b[k])
        assert e <= 1e-5, f"{k}: state vs recompute {e:.3e}"  # fp32 bar (in practice ~1e-7)


@pytest.mark.parametrize("B,n,C,T", [(9, 3, 48, 20), (33, 4, 128, 20), (11, 6, 64, 4), (4, 12, 64, 20),
                                     (3, 32, 64, 6)])
def test_saved_state_holds_the_denominators_of_every_iteration(B, n, C, T):
    """Replays the iterations on the CPU in float64 from the projection the forward saved:
    state[b, t, 0] are the row sums + eps of iteration t, state[b, t, 1] the column sums + eps
    (reference sinkhorn_knopp.cuh:38-120 adds eps to the sums)."""
    eps = 1e-6
    a = _fwd_bwd(B, n, C, torch.float32, T, eps, seed=3 * n + B, with_state=True)
    logits = a["alpha_res"] * a["P"].double()[:, 2 * n:] + a["b_res"].double().reshape(-1)
    m = torch.exp(logits).reshape(B, n, n)
    for t in range(T):
        rs = m.sum(2) + eps
        assert rel_err(a["sk"][:, t, 0], rs) <= 1e-5, ("row", t)
        m = m / rs[:, :, None]
        cs = m.sum(1) + eps
        assert rel_err(a["sk"][:, t, 1], cs) <= 1e-5, ("col", t)
        m = m / cs[:, None, :]
    assert rel_err(a["M"], m) <= 1e-5
