"""GPU parity: the HIP path, called through the C ABI, against the oracle.

fp32 tier:  max|got - ref| / max|ref| <= 1e-5 on y and every gradient (ref = oracle in fp64).
bf16 tier:  |got - ref| <= 2e-2 |ref| + 1e-2 elementwise (the stated tolerance) AND
            max|got - ref| / max|ref| <= 2e-2, so that small-magnitude gradients are not
            passed by the absolute term alone (ref = oracle in fp32 on the bf16-rounded inputs).
"""
import numpy as np
import pytest
import torch

from gpu_util import hip_dynamic, hip_static
from helpers import golden, rel_err
from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
BF16_RTOL, BF16_ATOL = 2e-2, 1e-2


def _check(got, ref, tier, what):
    ref = torch.as_tensor(ref).double()
    got = torch.as_tensor(got).double()
    e = rel_err(got, ref)
    if tier == "fp32":
        assert e <= FP32_TOL, f"{what}: rel err {e:.3e} > {FP32_TOL:.0e}"
    else:
        assert e <= BF16_RTOL, f"{what}: normalised err {e:.3e} > {BF16_RTOL}"
        bad = (got - ref).abs() > BF16_RTOL * ref.abs() + BF16_ATOL
        assert not bad.any(), f"{what}: {int(bad.sum())} elements outside rtol/atol"


def _t(a):
    return torch.from_numpy(np.asarray(a))


ALPHAS = ("alpha_pre", "alpha_post", "alpha_res")


def _alpha_term_sums(x, p, dy, T, eps, f_inject=None):
    """sum |term| of each alpha gradient, in float64.  d alpha_g = sum over samples and rows of the group
    of dL/dt * p is one scalar made of B n (or B n^2) terms of mixed sign; the oracle is run once more
    with each alpha spread out as a tensor of its own value per term, whose gradient holds the terms."""
    B, n = x.shape[0], x.shape[1]
    q = {k: torch.as_tensor(v) for k, v in p.items()}
    q["alpha_pre"] = q["alpha_pre"].double().reshape(()).expand(B, n).clone()
    q["alpha_post"] = q["alpha_post"].double().reshape(()).expand(B, n).clone()
    q["alpha_res"] = q["alpha_res"].double().reshape(()).expand(B, n, n).clone()
    _, g = nm.mhc_dynamic_fwd_bwd(x, q, dy, T, eps, f_inject=f_inject, dtype=torch.float64)
    return {k: float(g[k].abs().sum()) for k in ALPHAS if k in g}


def _check_alphas(g, g_ref, term_sums, tier):
    """Each of the three alpha gradients on its own: within the tier's relative tolerance of the sum of
    the absolute values of its terms (>= its own magnitude; equal to it when nothing cancels)."""
    tol = FP32_TOL if tier == "fp32" else BF16_RTOL
    for k in ALPHAS:
        if k not in g_ref:
            continue  # with an injected f nothing depends on alpha_pre
        got, ref = float(torch.as_tensor(g[k]).double()), float(torch.as_tensor(g_ref[k]).double())
        bar = tol * max(term_sums[k], abs(ref)) + (BF16_ATOL if tier == "bf16" else 0.0)
        assert abs(got - ref) <= bar, (f"d{k}: got {got:.9e}, oracle {ref:.9e}, |diff| {abs(got - ref):.3e} > "
                                       f"{bar:.3e} (sum |terms| {term_sums[k]:.3e})")


# ------------------------------------------------------------------------------------------------
# golden vectors written from the reference's own naive layers
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("tag", ["n4", "n16"])
def test_golden_functional_fp32(tag):
    g = golden("functional_" + tag)
    p = {k: _t(g[k]) for k in nm.DYN_PARAM_NAMES}
    y, grads = hip_dynamic(_t(g["x"]), p, _t(g["dy"]), int(g["T"]), float(g["eps"]))
    _check(y, g["y"], "fp32", "y")
    _check(grads["x"], g["dx"], "fp32", "dx")
    for k in nm.DYN_PARAM_NAMES:
        _check(grads[k], g["d" + k], "fp32", "d" + k)


@pytest.mark.parametrize("tag", ["n4", "n8", "n3"])
def test_golden_dynamic_module_fp32(tag):
    g = golden("dynamic_" + tag)
    p = {k: _t(g[k]) for k in nm.DYN_PARAM_NAMES}
    for k in ("phi_pre", "phi_post", "phi_res"):
        p[k] = p[k].t().contiguous()
    y, grads = hip_dynamic(_t(g["x"]), p, _t(g["dy"]), int(g["T"]), float(g["eps"]))
    _check(y, g["y"], "fp32", "y")
    _check(grads["x"], g["dx"], "fp32", "dx")
    for k in nm.DYN_PARAM_NAMES:
        ref = g["d" + k].T if k.startswith("phi") else g["d" + k]
        _check(grads[k], ref, "fp32", "d" + k)


@pytest.mark.parametrize("tag", ["n4", "n8"])
def test_golden_static_fp32(tag):
    g = golden("static_" + tag)
    p = {k: _t(g[k]) for k in nm.STATIC_PARAM_NAMES}
    y, grads = hip_static(_t(g["x"]), p, _t(g["dy"]), int(g["T"]), float(g["eps"]))
    _check(y, g["y"], "fp32", "y")
    _check(grads["x"], g["dx"], "fp32", "dx")
    for k in nm.STATIC_PARAM_NAMES:
        _check(grads[k], g["d" + k], "fp32", "d" + k)


# ------------------------------------------------------------------------------------------------
# seeded inputs against the oracle: small shapes, ragged shapes, every layout of the kernels
# ------------------------------------------------------------------------------------------------
def _rand_params(p, n, C, seed=7):
    """Move every parameter away from its init value so that no gradient path is trivially zero."""
    g = torch.Generator().manual_seed(seed)
    p = dict(p)
    p["w"] = 1.0 + 0.3 * torch.randn(C, generator=g)
    p["b_pre"] = 0.3 * torch.randn(n, generator=g)
    p["b_post"] = 0.3 * torch.randn(n, generator=g)
    p["b_res"] = 0.5 * torch.randn(n, n, generator=g)
    p["alpha_pre"] = torch.tensor(0.05)
    p["alpha_post"] = torch.tensor(-0.03)
    p["alpha_res"] = torch.tensor(0.04)
    return p


DYN_SHAPES = [
    (32, 4, 1280), (5, 4, 64), (1, 4, 128), (3, 2, 40), (2, 3, 20), (7, 1, 36),
    (16, 8, 256), (3, 6, 72), (4, 16, 64), (3, 12, 40), (4, 32, 64), (2, 24, 104), (2, 32, 1040),
    # n > 8 in float32: several tiles and a ragged last slice for the fp32 matrix-core products, and
    # a row length that is not a multiple of 4 (scalar kernels)
    (130, 12, 36), (3, 9, 10),
    # a batch far beyond the CU count, a row too long for the fused forward kernel, odd expansion rates
    (2100, 4, 32), (2, 4, 4400), (3, 17, 24), (2, 31, 40),
]


@pytest.mark.parametrize("B,n,C", DYN_SHAPES)
@pytest.mark.parametrize("inject", [False, True])
def test_dynamic_fp32_vs_oracle(B, n, C, inject):
    x, dy, f, p = nm.make_dynamic_inputs(B, n, C, with_f=inject)
    p = _rand_params(p, n, C)
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=torch.float64)
    y, g = hip_dynamic(x, p, dy, T, eps, f_inject=f)
    _check(y, y_ref, "fp32", "y")
    assert set(g_ref) <= set(g), f"missing gradients {set(g_ref) - set(g)}"
    if n > 1:
        _check_alphas(g, g_ref, _alpha_term_sums(x, p, dy, T, eps, f), "fp32")
    for k, ref in g_ref.items():
        if n > 1 and k in ALPHAS:
            continue
        if n == 1 and k in ("phi_pre", "b_pre", "alpha_pre"):
            # one stream: f = RMSNorm(H_pre x) w does not depend on H_pre except through eps, so
            # the true gradient is O(eps) (times the batch) and a relative comparison is meaningless
            assert float((g[k].double() - torch.as_tensor(ref).double()).abs().max()) < 1e-4
            continue
        _check(g[k], ref, "fp32", "d" + k)


@pytest.mark.parametrize("n", [16, 32])
def test_sinkhorn_backward_round_off_does_not_grow_with_the_iteration_count(n):
    """n > 8, fp32: the gradient of the Sinkhorn logits stays at a few 1e-7 of the float64 oracle from
    20 to 256 iterations (it grew by ~2e-8 per iteration while the forward formed its denominators
    with a fused multiply-add; tests/test_sinkhorn_roundoff_model.py holds the CPU model)."""
    B, C, eps = 2, 8, 1e-6
    for T in (20, 256):
        x, dy, f, p = nm.make_dynamic_inputs(B, n, C, with_f=False)
        p = _rand_params(p, n, C)
        _, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, dtype=torch.float64)
        _, g = hip_dynamic(x, p, dy, T, eps)
        for k in ("b_res", "phi_res"):
            e = rel_err(g[k], g_ref[k])
            assert e <= 1e-6, f"d{k} at T={T}: rel err {e:.3e}"


@pytest.mark.parametrize("B,n,C,T", [(2, 4, 16, 256), (3, 8, 16, 256), (2, 5, 16, 256), (2, 16, 8, 256), (2, 32, 8, 256),
                                     (3, 8, 64, 60)])
@pytest.mark.parametrize("dyn", [True, False])
def test_largest_iteration_counts(B, n, C, T, dyn):
    """The largest accepted iteration count of every Sinkhorn layout (LDS above 64 KB per workgroup):
    forward and exact backward against the float64 oracle."""
    eps = 1e-6
    if dyn:
        x, dy, f, p = nm.make_dynamic_inputs(B, n, C, with_f=False)
        p = _rand_params(p, n, C)
        y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, dtype=torch.float64)
        y, g = hip_dynamic(x, p, dy, T, eps)
    else:
        x, dy, f, p = nm.make_static_inputs(B, n, C, with_f=False)
        y_ref, g_ref = nm.mhc_static_fwd_bwd(x, p, dy, T, eps, dtype=torch.float64)
        y, g = hip_static(x, p, dy, T, eps)
    _check(y, y_ref, "fp32", "y")
    for k, ref in g_ref.items():
        _check(g[k], ref, "fp32", "d" + k)


@pytest.mark.parametrize("B,n,C", [(32, 4, 1280), (5, 4, 64), (16, 8, 256), (3, 6, 72), (4, 16, 64),
                                   (4, 32, 64), (2, 32, 1040), (3, 4, 20),
                                   # more than 128 samples with a wide projection: several sample
                                   # blocks / groups in the projection kernels
                                   (160, 20, 64), (130, 32, 136),
                                   # two chunks per thread with a ragged chunk count and a partial sample tile;
                                   # n between the tile sizes; one sample; C not a multiple of 8 with n > 8
                                   (33, 4, 2568), (3, 12, 40), (2, 24, 104), (1, 32, 128), (3, 20, 36),
                                   # a batch far beyond the CU count (several samples per workgroup, batch
                                   # splits), a row too long for the fused forward kernel, odd expansion rates
                                   (4100, 4, 64), (2, 4, 8200), (3, 17, 24), (2, 31, 40), (600, 8, 64),
                                   # wide projection with batch splits and many sample blocks per split
                                   (4000, 20, 32),
                                   # two chunks per thread in the fused forward with 8 x 8 coefficients
                                   (3, 8, 2568), (2, 5, 4096)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_dynamic_bf16_vs_oracle(B, n, C, out_dtype):
    x, dy, _, p = nm.make_dynamic_inputs(B, n, C, bf16_round=True)
    p = _rand_params(p, n, C)
    for k in ("w", "phi_pre", "phi_post", "phi_res"):
        p[k] = p[k].bfloat16().float()
    if out_dtype == torch.float32:
        dy_used = dy
    else:
        dy_used = dy.bfloat16().float()
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy_used, T, eps, dtype=torch.float32)
    y, g = hip_dynamic(x, p, dy_used, T, eps, act_dtype=torch.bfloat16, out_dtype=out_dtype,
                       w_dtype=torch.bfloat16)
    _check(y, y_ref, "bf16", "y")
    for k, ref in g_ref.items():
        _check(g[k], ref, "bf16", "d" + k)


# n <= 8 with bf16 activations: the channel sums of the backward are Gram matrices built from 4x4
# matrix-core products (one to eight streams, one 128-channel step with and without a tail, one and two
# column parts).
# The small parameter gradients only see exact bf16 products summed in fp32, so they are held to a
# bound far below the bf16 tolerance: a dropped remainder term or a misplaced Gram entry fails it.
@pytest.mark.parametrize("B,n,C", [(5, 1, 8), (3, 2, 136), (6, 3, 1032), (40, 4, 1288), (7, 4, 128),
                                   (1100, 4, 1024), (6, 5, 136), (4, 7, 128), (9, 8, 1288), (70, 6, 1024)])
@pytest.mark.parametrize("inject", [False, True])
@pytest.mark.parametrize("w_dtype", [torch.bfloat16, torch.float32])
def test_bf16_small_n_coefficient_gradients_are_tight(B, n, C, inject, w_dtype):
    x, dy, f, p = nm.make_dynamic_inputs(B, n, C, bf16_round=True, with_f=inject)
    p = _rand_params(p, n, C)
    for k in ("phi_pre", "phi_post", "phi_res") + (("w",) if w_dtype == torch.bfloat16 else ()):
        p[k] = p[k].bfloat16().float()
    if f is not None:
        f = f.bfloat16().float()
    dy = dy.bfloat16().float()
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=torch.float64)
    y, g = hip_dynamic(x, p, dy, T, eps, f_inject=f, act_dtype=torch.bfloat16, out_dtype=torch.bfloat16,
                       w_dtype=w_dtype)
    _check(y, y_ref, "bf16", "y")
    _check(g["x"], g_ref["x"], "bf16", "dx")
    for k in ("b_pre", "b_post", "b_res", "alpha_pre", "alpha_post", "alpha_res"):
        if inject and k in ("b_pre", "alpha_pre"):
            continue  # an injected f does not depend on H_pre
        if n == 1 and k in ("b_pre", "alpha_pre"):
            assert float((g[k].double() - g_ref[k].double()).abs().max()) < 1e-4  # O(eps), see test_dynamic_fp32_vs_oracle
            continue
        e = rel_err(g[k], g_ref[k])
        assert e <= 2e-4, f"d{k}: normalised err {e:.3e}"


@pytest.mark.parametrize("B,n,C", [(16, 4, 256), (8, 8, 128), (4, 16, 64), (3, 32, 72), (5, 32, 1040),
                                   (5, 4, 2568), (3, 7, 2176),
                                   # 128 samples and more: the channel sums run on the matrix cores
                                   (130, 4, 264), (128, 7, 136), (300, 3, 1288), (129, 8, 2048),
                                   # 1024 samples and more with n <= 4: the dx kernel takes four samples per workgroup
                                   (1100, 4, 72)])
@pytest.mark.parametrize("inject", [False, True])
def test_static_bf16_vs_oracle(B, n, C, inject):
    """Static H with bf16 activations: the shared-coefficient mode of the bf16 kernels."""
    x, dy, f, p = nm.make_static_inputs(B, n, C, with_f=inject)
    x, dy = x.bfloat16().float(), dy.bfloat16().float()
    f = None if f is None else f.bfloat16().float()
    p["w"] = (1.0 + 0.3 * torch.randn(C, generator=torch.Generator().manual_seed(3))).bfloat16().float()
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_static_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=torch.float32)
    y, g = hip_static(x, p, dy, T, eps, f_inject=f, act_dtype=torch.bfloat16, w_dtype=torch.bfloat16)
    _check(y, y_ref, "bf16", "y")
    for k, ref in g_ref.items():
        _check(g[k], ref, "bf16", "d" + k)


@pytest.mark.parametrize("B,n,C", [(32, 4, 1280), (3, 4, 20), (8, 8, 128), (4, 16, 64), (3, 32, 72), (1030, 3, 40)])
@pytest.mark.parametrize("inject", [False, True])
def test_static_fp32_vs_oracle(B, n, C, inject):
    x, dy, f, p = nm.make_static_inputs(B, n, C, with_f=inject)
    p["w"] = 1.0 + 0.3 * torch.randn(C, generator=torch.Generator().manual_seed(3))
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_static_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=torch.float64)
    y, g = hip_static(x, p, dy, T, eps, f_inject=f)
    _check(y, y_ref, "fp32", "y")
    for k, ref in g_ref.items():
        _check(g[k], ref, "fp32", "d" + k)


# ------------------------------------------------------------------------------------------------
# the benchmark configurations at full size
# ------------------------------------------------------------------------------------------------
def test_config1_static_fp32_full_size():
    B, n, C = 320, 4, 1280
    x, dy, f, p = nm.make_static_inputs(B, n, C, with_f=True)
    T, eps = 20, 1e-6
    for inj in (None, f):
        y_ref, g_ref = nm.mhc_static_fwd_bwd(x, p, dy, T, eps, f_inject=inj, dtype=torch.float64)
        y, g = hip_static(x, p, dy, T, eps, f_inject=inj)
        _check(y, y_ref, "fp32", "y")
        for k, ref in g_ref.items():
            _check(g[k], ref, "fp32", "d" + k)


@pytest.mark.parametrize("B,n,C", [(320, 4, 1280), (1280, 4, 2560), (256, 8, 1280), (128, 32, 1280)])
@pytest.mark.parametrize("inject", [False, True])
def test_configs_2_to_5_bf16_full_size(B, n, C, inject):
    x, dy, f, p = nm.make_dynamic_inputs(B, n, C, bf16_round=True, with_f=inject)
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=torch.float32)
    y, g = hip_dynamic(x, p, dy, T, eps, f_inject=f, act_dtype=torch.bfloat16,
                       out_dtype=torch.bfloat16, w_dtype=torch.bfloat16)
    _check(y, y_ref, "bf16", "y")
    for k, ref in g_ref.items():
        _check(g[k], ref, "bf16", "d" + k)
    # The float32 gradients of this tier are float32 sums of products of the rounded inputs (the
    # coefficient gradients enter the matrix cores as bf16 value + remainder): they sit at a few 1e-6 of
    # the oracle, far inside the tier's tolerance, and a dropped low-order term would show here.
    for k in ("phi_pre", "phi_post", "phi_res", "b_pre", "b_post", "b_res"):
        if k in g_ref:
            e = rel_err(torch.as_tensor(g[k]).double(), torch.as_tensor(g_ref[k]).double())
            assert e <= 1e-4, f"d{k}: rel err {e:.3e} > 1e-4"


def test_config2_fp32_full_size():
    """The headline shape in the fp32 tier (1e-5)."""
    B, n, C = 320, 4, 1280
    x, dy, _, p = nm.make_dynamic_inputs(B, n, C)
    T, eps = 20, 1e-6
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, dtype=torch.float64)
    y, g = hip_dynamic(x, p, dy, T, eps)
    _check(y, y_ref, "fp32", "y")
    sums = _alpha_term_sums(x, p, dy, T, eps)
    _check_alphas(g, g_ref, sums, "fp32")
    for k in ALPHAS:  # reported on its own: error relative to the gradient itself and to its terms
        got, ref = float(g[k]), float(g_ref[k])
        print(f"d{k}: {got:.7e} (oracle {ref:.7e}) rel {abs(got - ref) / abs(ref):.2e}, of sum|terms| {abs(got - ref) / sums[k]:.2e}")
    for k, ref in g_ref.items():
        if k not in ALPHAS:
            _check(g[k], ref, "fp32", "d" + k)


def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        n = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 31, 32]))
        B = int(rng.choice([1, 2, 3, 5, 17, 33, 64, 129, 260]))
        unit = int(rng.choice([1, 2, 4, 8]))
        C = unit * int(rng.integers(1, 40))
        if n * C * B > 600_000:   # keep the float64 oracle quick
            B = max(1, 600_000 // (n * C))
        T = int(rng.choice([0, 1, 3, 20]))
        cases.append((B, n, C, T, bool(rng.integers(2)), bool(rng.integers(2)), bool(rng.integers(2))))
    return cases


# two cases kept from wider sweeps: a static Sinkhorn gradient that plain float32 PyTorch misses by
# 7.5e-5, and a single-channel layer with 32 streams
_KEPT_CASES = [(260, 2, 100, 20, False, False, False), (1, 32, 1, 1, True, False, False),
               (3, 32, 1, 1, True, False, False)]
# long rows, up to the largest accepted hidden size (a wider sweep over C = 8192 .. 32768, n = 1 .. 32, both
# tiers and both coefficient modes passed as well)
_KEPT_CASES += [(3, 4, 32768, 20, True, True, False), (2, 32, 32768, 20, True, True, False),
                (3, 8, 20000, 20, True, True, False), (33, 1, 32768, 20, False, False, False),
                (3, 9, 16384, 20, True, False, False), (3, 4, 12296, 20, False, True, False)]
# 11 <= n <= 18 with a large batch: the two projection-backward products as launches of their own, with batch
# splits (the finalize launch sums the dphi copies) and, in the second case, without dw
_KEPT_CASES += [(2000, 12, 32, 20, True, True, False), (3000, 16, 32, 20, True, True, True)]
# very large batches of short rows: the channel sums and the coefficient backward as two launches (n <= 4)
_KEPT_CASES += [(6100, 4, 128, 20, True, True, False), (6500, 3, 256, 20, True, True, True)]


@pytest.mark.parametrize("B,n,C,T,dyn,bf16,inject", _random_cases(40, seed=2024) + _KEPT_CASES)
def test_random_shapes_vs_oracle(B, n, C, T, dyn, bf16, inject):
    """Seeded sweep over shapes, iteration counts (0 and 1 included), both coefficient modes, both
    precision tiers and both views, against the oracle."""
    eps = 1e-6
    act = torch.bfloat16 if bf16 else torch.float32
    tier = "bf16" if bf16 else "fp32"
    make = nm.make_dynamic_inputs if dyn else nm.make_static_inputs
    x, dy, f, p = make(B, n, C, with_f=inject)
    if dyn:
        p = _rand_params(p, n, C)
    if bf16:
        x, dy = x.bfloat16().float(), dy.bfloat16().float()
        f = None if f is None else f.bfloat16().float()
        for k in ("w", "phi_pre", "phi_post", "phi_res"):
            if k in p:
                p[k] = p[k].bfloat16().float()
    ref_dtype = torch.float32 if bf16 else torch.float64
    if dyn:
        y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=ref_dtype)
        y, g = hip_dynamic(x, p, dy, T, eps, f_inject=f, act_dtype=act, out_dtype=act,
                           w_dtype=act)
    else:
        y_ref, g_ref = nm.mhc_static_fwd_bwd(x, p, dy, T, eps, f_inject=f, dtype=ref_dtype)
        y, g = hip_static(x, p, dy, T, eps, f_inject=f, act_dtype=act, out_dtype=act, w_dtype=act)
    _check(y, y_ref, tier, "y")
    assert set(g_ref) <= set(g), f"missing gradients {set(g_ref) - set(g)}"
    per_alpha = dyn and n > 1 and C > 1
    if per_alpha:
        _check_alphas(g, g_ref, _alpha_term_sums(x, p, dy, T, eps, f), tier)
    for k, ref in g_ref.items():
        if per_alpha and k in ALPHAS:
            continue
        tiny = ("phi_pre", "b_pre", "alpha_pre", "H_pre") + (("phi_res", "b_res", "alpha_res", "H_res") if T > 0 and n == 1 else ())
        # one channel: the inner RMSNorm maps the aggregate to its sign, so f does not depend on H_pre
        # either (except through eps)
        if (n == 1 or (C == 1 and not inject)) and k in tiny:
            # one stream: f does not depend on H_pre except through eps, and the 1 x 1 Sinkhorn output
            # (after at least one iteration) is 1 / (1 + O(eps)) whatever its logit, so these gradients are O(eps) (bf16: rounding
            # noise of that size) and a relative comparison is meaningless
            # (their rounding noise grows with the row length: plain float32 PyTorch is 1.5e-4 off at C = 32768)
            bar = 1e-2 if bf16 else 1e-4 * max(1.0, C / 1024)
            assert float((g[k].double() - torch.as_tensor(ref).double()).abs().max()) < bar, k
            continue
        if C == 1 and not inject and not bf16 and k == "x":
            # one channel: the backward of the inner RMSNorm is the difference of two terms that are
            # equal up to eps / q^2, and the kernels rebuild the aggregate in two launches with
            # different summation orders, so the difference carries their rounding (seen: 4.6e-5 of
            # |dx| with 32 streams); a hidden size of 1 is a degenerate layer
            assert rel_err(torch.as_tensor(g[k]).double().cpu(), torch.as_tensor(ref).double()) <= 2e-4, k
            continue
        _check(g[k], ref, tier, "d" + k)


@pytest.mark.parametrize("bf16", [False, True])
def test_more_than_65535_samples_with_more_than_8_streams(bf16):
    """The reference launches one block per sample on the first grid dimension and has no bound on the
    batch (src/csrc/kernels/sinkhorn_knopp.cuh:1015-1045); neither do the n > 8 kernels here."""
    B, n, C, T, eps = 70001, 9, 8, 3, 1e-6
    x, dy, _, p = nm.make_dynamic_inputs(B, n, C, bf16_round=bf16)
    p = _rand_params(p, n, C)
    act = torch.bfloat16 if bf16 else torch.float32
    if bf16:
        for k in ("w", "phi_pre", "phi_post", "phi_res"):
            p[k] = p[k].bfloat16().float()
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x, p, dy, T, eps, dtype=torch.float32 if bf16 else torch.float64)
    y, g = hip_dynamic(x, p, dy, T, eps, act_dtype=act, out_dtype=act, w_dtype=act)
    tier = "bf16" if bf16 else "fp32"
    _check(y, y_ref, tier, "y")
    _check(g["x"], g_ref["x"], tier, "dx")
    _check_alphas(g, g_ref, _alpha_term_sums(x, p, dy, T, eps), tier)
    for k in ("phi_res", "b_res", "w"):
        _check(g[k], g_ref[k], tier, "d" + k)
