"""The two n <= 8 bf16 backward paths of the library against the oracle and against each other, through
the C ABI of the tuning build (the launch heuristic picks one of them by batch size; here each is
forced on the same inputs):

  resident  one workgroup per sample keeps dy and x in registers (channel sums, coefficient backward,
            mixing part of dx), then a column-slab kernel completes dx and finishes dphi and the
            batch sums                                         (bwd_resident.hip, proj_bwd_addx.hip)
  tiled     channel sums, then the slab kernel (n <= 4) or projection backward + dx kernel, then the
            batch-sum launch

The same is done for wide projections (n > 18), where the library runs the dx workgroups that need no
result of the coefficient backward beside it in one launch and lets the dP phi kernel complete dx
(four launches), against the five-launch order that the tuning build can still force.

Tolerances: the bf16 tier of test_gpu_parity.py against the oracle (fp32 on the bf16-rounded inputs);
between the paths the parameter gradients (exact bf16 products summed in fp32 on both sides) agree to
2e-4 of their largest entry, dx to two bf16 roundings.
"""
import pytest
import torch

from helpers import pack_dynamic_grads, rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu

K_RESIDENT, K_WIDE_DX_BESIDE = 7, 8
T_ITERS, EPS = 20, 1e-6


def _step(B, n, C, inject, w_f32):
    import bench
    from mhc._lib import tuning_lib

    cfg = dict(kind="dynamic", B=B, n=n, C=C, dtype="bf16", bwd=True)
    st = bench.Step(cfg, "K" if inject else "L", torch, lib=tuning_lib())
    # move the parameters away from their init values so that no gradient path is trivially zero
    g = torch.Generator().manual_seed(B * 7 + n * 131 + C)
    p = st.host["p"]
    p["w"] = (1.0 + 0.3 * torch.randn(C, generator=g))
    if not w_f32:
        p["w"] = p["w"].bfloat16().float()
    p["b_pre"], p["b_post"] = 0.3 * torch.randn(n, generator=g), 0.3 * torch.randn(n, generator=g)
    p["b_res"] = 0.5 * torch.randn(n, n, generator=g)
    p["alpha_pre"], p["alpha_post"], p["alpha_res"] = torch.tensor(0.05), torch.tensor(-0.03), torch.tensor(0.04)
    st.w = p["w"].to(torch.float32 if w_f32 else torch.bfloat16).cuda()
    st.bias.copy_(torch.cat([p["b_pre"], p["b_post"], p["b_res"].reshape(-1)]))
    st.alpha.copy_(torch.stack([p["alpha_pre"], p["alpha_post"], p["alpha_res"]]))
    return st


def _grads(st):
    out = {k: getattr(st, k).float().cpu() for k in ("dx", "dphi", "dbias", "dalpha")}
    if st.df is not None:
        out["df"] = st.df.float().cpu()
    else:
        out["dw"] = st.dw.float().cpu()
    return out


SHAPES = [(5, 4, 64), (1, 4, 128), (3, 2, 40), (2, 3, 24), (7, 1, 136), (33, 4, 1288), (320, 4, 1280), (9, 4, 640),
          (130, 4, 2560), (16, 8, 256), (3, 6, 72), (9, 8, 1288), (70, 5, 1024), (257, 8, 136), (300, 7, 512),
          (1100, 8, 128), (1030, 5, 264)]   # short rows, large batch: where the default takes the tiled path for n > 4


def _both_paths(key, names, B, n, C, inject, w_f32):
    """Backward of one step with tuning hook `key` at 1 and at 2 (names = what the two settings are called):
    each against the oracle, then against each other."""
    st = _step(B, n, C, inject, w_f32)
    lib = st.lib
    h = st.host
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(h["x"], h["p"], h["dy"], T_ITERS, EPS, f_inject=h["f"], dtype=torch.float32)
    dphi_ref, dbias_ref, dalpha_ref = pack_dynamic_grads(
        {k: g_ref.get(k, torch.zeros_like(torch.as_tensor(h["p"][k]))) for k in nm.DYN_PARAM_NAMES if k != "w"}, n)
    ref = dict(dx=g_ref["x"], dphi=dphi_ref, dbias=dbias_ref, dalpha=dalpha_ref)
    if inject:
        ref["df"] = g_ref["f"]
    else:
        ref["dw"] = g_ref["w"]
    st.forward()
    got = {}
    try:
        for mode, name in ((1, names[0]), (2, names[1])):
            assert lib.mhc_tuning_set(key, mode) == 0
            for t in (st.dx, st.dphi, st.dbias, st.dalpha, st.dw) + ((st.df,) if st.df is not None else ()):
                t.fill_(float("nan"))
            st.backward()
            torch.cuda.synchronize()
            got[name] = _grads(st)
    finally:
        lib.mhc_tuning_set(key, 0)
    for name, g in got.items():
        for k, r in ref.items():
            assert torch.isfinite(g[k]).all(), f"{name}: {k} not finite"
            if n == 1 and not inject and k in ("dphi", "dbias", "dalpha"):
                continue  # one stream: the pre entries are O(eps) (see test_gpu_parity.py); compared between the paths below
            e = rel_err(g[k], r)
            assert e <= 2e-2, f"{name}: {k} normalised err {e:.3e}"
            bad = (g[k].double() - r.double()).abs() > 2e-2 * r.double().abs() + 1e-2
            assert not bad.any(), f"{name}: {k} {int(bad.sum())} elements outside rtol/atol"
    for k in ("dphi", "dbias", "dalpha") + (() if inject else ("dw",)):
        e = rel_err(got[names[1]][k], got[names[0]][k])
        assert e <= 2e-4, f"{k} {names[1]} vs {names[0]}: {e:.3e}"
    e = rel_err(got[names[1]]["dx"], got[names[0]]["dx"])
    assert e <= 1.6e-2, f"dx {names[1]} vs {names[0]}: {e:.3e}"


@pytest.mark.parametrize("B,n,C", SHAPES)
@pytest.mark.parametrize("inject", [False, True])
@pytest.mark.parametrize("w_f32", [False, True])
def test_resident_and_tiled_backward(B, n, C, inject, w_f32):
    if inject and w_f32:
        pytest.skip("w is unused with an injected f")
    _both_paths(K_RESIDENT, ("tiled", "resident"), B, n, C, inject, w_f32)


WIDE_SHAPES = [(128, 32, 1280), (5, 32, 64), (1, 19, 128), (130, 20, 136), (33, 27, 264), (260, 32, 8), (64, 24, 2056),
               (3000, 20, 8)]


@pytest.mark.parametrize("B,n,C", WIDE_SHAPES)
@pytest.mark.parametrize("inject", [False, True])
@pytest.mark.parametrize("w_f32", [False, True])
def test_wide_backward_dx_beside_the_coefficient_launch(B, n, C, inject, w_f32):
    if inject and w_f32:
        pytest.skip("w is unused with an injected f")
    _both_paths(K_WIDE_DX_BESIDE, ("five launches", "four launches"), B, n, C, inject, w_f32)
