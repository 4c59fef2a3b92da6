"""Runtime properties of the C ABI calls: HIP-graph capture and replay, bit-exact determinism,
re-entrancy across streams with separate workspaces, and the compute_dtype option of MHCLayer."""
import pytest
import torch

from oracle import naive_mhc as nm

pytestmark = pytest.mark.gpu


def _bf16_step(B, n, C, lib=None):
    import bench

    cfg = dict(kind="dynamic", B=B, n=n, C=C, dtype="bf16", bwd=True)
    return bench.Step(cfg, "L", torch, lib=lib)


@pytest.mark.parametrize("B,n,C", [(96, 4, 512), (40, 8, 256), (24, 32, 256)])
def test_graph_replay_matches_eager_and_is_deterministic(B, n, C):
    """Forward + backward captured in one HIP graph; three replays, with unrelated eager work and
    synchronisations between them, must each reproduce the eager results bit for bit."""
    st = _bf16_step(B, n, C)
    outs = lambda: [t.clone() for t in (st.y, st.dx, st.dw, st.dphi, st.dbias, st.dalpha)]
    st.step()
    torch.cuda.synchronize()
    eager = outs()
    st.step()
    torch.cuda.synchronize()
    for a, b in zip(eager, outs()):
        assert torch.equal(a, b), "two eager runs differ"
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        st.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st.step()
    scratch = torch.zeros(1 << 20, device="cuda")
    for rep in range(3):
        for t in (st.y, st.dx, st.dw, st.dphi, st.dbias, st.dalpha):
            t.fill_(float("nan"))
        scratch.add_(1.0).sum().item()  # eager work + a host sync between replays
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "dx", "dw", "dphi", "dbias", "dalpha"), eager, outs()):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager result"


@pytest.mark.parametrize("shapes", [((64, 4, 512), (48, 4, 1024)), ((24, 32, 128), (16, 32, 256))])
def test_two_streams_with_separate_workspaces(shapes):
    """Two layer calls in flight on two streams, each with its own workspace, give the results of
    running them one after the other."""
    a, b = _bf16_step(*shapes[0]), _bf16_step(*shapes[1])
    for s in (a, b):
        s.step()
    torch.cuda.synchronize()
    ref = [[t.clone() for t in (s.y, s.dx, s.dphi)] for s in (a, b)]
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(5):
        with torch.cuda.stream(s1):
            a.step()
        with torch.cuda.stream(s2):
            b.step()
    torch.cuda.synchronize()
    for s, r in zip((a, b), ref):
        for got, want in zip((s.y, s.dx, s.dphi), r):
            assert torch.equal(got, want)


@pytest.mark.parametrize("B,n,C", [(70, 8, 512), (33, 10, 256), (64, 12, 256), (300, 16, 128)])
def test_projection_backward_products_apart_match_one_launch(B, n, C):
    """dphi = dP^T x and dP phi as two launches around the dx kernel (the default from n = 11 on) against
    both in one launch, each forced through the experiment hook: same gradients bit for bit."""
    from mhc._lib import tuning_lib

    lib = tuning_lib()  # the build of the library whose launch heuristics can be overridden
    st = _bf16_step(B, n, C, lib)
    outs = (st.dx, st.dw, st.dphi, st.dbias, st.dalpha)
    try:
        assert lib.mhc_tuning_set(4, 1) == 0  # batch sums in their own launch both times
        res = []
        for mode in (1, 2):
            assert lib.mhc_tuning_set(5, mode) == 0
            for t in outs:
                t.fill_(float("nan"))
            st.step()
            torch.cuda.synchronize()
            res.append([t.clone() for t in outs])
        for name, a, b in zip(("dx", "dw", "dphi", "dbias", "dalpha"), *res):
            assert torch.isfinite(a).all(), name
            assert torch.equal(a, b), name
    finally:
        lib.mhc_tuning_set(4, 0)
        lib.mhc_tuning_set(5, 0)


@pytest.mark.parametrize("B,n,C", [(40, 32, 256), (33, 20, 256), (128, 24, 64), (33, 12, 256), (70, 16, 128)])
def test_batch_sums_inside_the_dphi_launch_match_the_separate_launch(B, n, C):
    """From n = 11 on: dw, dbias and dalpha summed by extra workgroups of the dphi launch (the default)
    against the same sums as a launch of their own (forced through the experiment hook), eagerly with
    poisoned outputs and under graph replay."""
    from mhc._lib import tuning_lib

    lib = tuning_lib()  # the build of the library whose launch heuristics can be overridden
    st = _bf16_step(B, n, C, lib)
    outs = (st.dx, st.dw, st.dphi, st.dbias, st.dalpha)
    grads = lambda: [t.clone() for t in outs]

    def check(what):
        for name, a, b in zip(("dx", "dw", "dphi", "dbias", "dalpha"), ref, grads()):
            if name in ("dx", "dphi"):
                assert torch.equal(a, b), f"{what}: {name}"
            else:  # float64 sums of the same float32 terms, grouped differently: equal up to the final rounding
                torch.testing.assert_close(b, a, rtol=1e-6, atol=0, msg=f"{what}: {name}")

    try:
        assert lib.mhc_tuning_set(4, 1) == 0
        st.step()
        torch.cuda.synchronize()
        ref = grads()
        assert lib.mhc_tuning_set(4, 0) == 0
        for rep in range(3):
            for t in outs:
                t.fill_(float("nan"))
            st.step()
            torch.cuda.synchronize()
            check(f"run {rep}")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            st.step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            st.step()
        scratch = torch.zeros(1 << 20, device="cuda")
        for rep in range(3):
            for t in outs:
                t.fill_(float("nan"))
            scratch.add_(1.0).sum().item()  # eager work + a host sync between replays
            graph.replay()
            torch.cuda.synchronize()
            check(f"replay {rep}")
    finally:
        lib.mhc_tuning_set(4, 0)


def _module_grads(layer, x, dy):
    layer.zero_grad()
    xg = x.clone().requires_grad_(True)
    y = layer(xg)
    y.backward(dy.to(y.dtype))
    g = {"x": xg.grad}
    g.update({k: p.grad for k, p in layer.named_parameters()})
    return y, g


@pytest.mark.parametrize("B,n,C", [(16, 4, 256), (320, 4, 1280), (37, 3, 72), (40, 8, 264), (2000, 4, 64), (6, 12, 64)])
def test_compute_dtype_bf16_on_float32_activations(B, n, C):
    """MHCLayer(compute_dtype=bfloat16) on float32 activations - the reference's default contract (float32 in
    and out around a bf16 kernel path, ops.py:129,404, bindings.cu:421-423).  Where the kernels load
    float32 storage themselves (n <= 8) no cast runs; elsewhere (n > 8) the operator casts.  Either way the results stay float32 and agree with the oracle on the bf16-rounded
    activations at the bf16 tolerance, and with the same layer fed the bf16-rounded activations."""
    from helpers import rel_err
    from mhc import MHCLayer
    from mhc._lib import lib
    from oracle import naive_mhc as nm

    T, eps = 20, 1e-6
    torch.manual_seed(3)
    layer = MHCLayer(C, n, sinkhorn_iters=T, eps=eps, use_dynamic_h=True, compute_dtype=torch.bfloat16).cuda()
    with torch.no_grad():  # coefficients that depend on x, parameters as the bf16 kernels see them
        for k in ("alpha_pre", "alpha_post", "alpha_res"):
            getattr(layer, k).fill_(0.3)
        for k in ("phi_pre", "phi_post", "phi_res"):
            getattr(layer, k).copy_(getattr(layer, k).bfloat16().float())
        layer.b_res.copy_(0.3 * torch.randn(n, n))
    x = torch.randn(B, n, C, device="cuda")
    dy = torch.randn(B, n, C, device="cuda")
    in_kernel = bool(lib.mhc_layer_dynamic_accepts_f32_as_bf16(B, n, C, T))
    assert in_kernel == (n <= 8)
    y, g = _module_grads(layer, x, dy)
    assert y.dtype == torch.float32 and g["x"].dtype == torch.float32
    # the oracle on the rounded activations
    p = {k: v.detach().float().cpu() for k, v in layer.named_parameters()}
    p["w"] = p.pop("rmsnorm_weight")
    # (the incoming gradient is an activation too: the kernels that take float32 storage round it like x,
    # and the cast path rounds it with a cast of its own before the backward call)
    dy_seen = dy.bfloat16().float()
    y_ref, g_ref = nm.mhc_dynamic_fwd_bwd(x.bfloat16().float().cpu(), p, dy_seen.cpu(), T, eps, dtype=torch.float32)
    g_ref["rmsnorm_weight"] = g_ref.pop("w")

    def check(got, ref, what):
        got, ref = got.detach().float().cpu().double(), torch.as_tensor(ref).double()
        assert rel_err(got, ref) <= 2e-2, f"{what}: {rel_err(got, ref):.3e}"
        bad = (got - ref).abs() > 2e-2 * ref.abs() + 1e-2
        assert not bad.any(), f"{what}: {int(bad.sum())} elements outside rtol/atol"

    check(y, y_ref, "y")
    for k, ref in g_ref.items():
        check(g[k], ref, "d" + k)
    # the same layer on activations that were rounded beforehand
    plain = MHCLayer(C, n, sinkhorn_iters=T, eps=eps, use_dynamic_h=True).cuda()
    plain.load_state_dict(layer.state_dict())
    y2, g2 = _module_grads(plain, x.bfloat16(), dy_seen)
    assert rel_err(y, y2) <= 1e-2
    for k in g:
        assert rel_err(g[k], g2[k]) <= 2e-2, k


@pytest.mark.parametrize("n,C,src,dst", [
    (4, 64, torch.float32, torch.bfloat16),      # small: one chunk per thread
    (3, 20, torch.float32, torch.bfloat16),      # lengths that are no multiple of 8: element-wise kernel
    (16, 520, torch.float32, torch.bfloat16),    # 2.4 M elements: the streaming kernel, ragged last round
    (32, 1280, torch.float32, torch.bfloat16),   # the largest benchmark shape (44.6 M elements)
    (16, 520, torch.float32, torch.float32),
    (16, 520, torch.bfloat16, torch.bfloat16),
])
def test_parameter_gather_is_the_rounded_concatenation(n, C, src, dst):
    """mhc_pack_dynamic_params: phi is the row concatenation [pre | post | res] converted once (round to
    nearest even for bfloat16), the biases and alphas are copied; every element, bit for bit."""
    from mhc import _lib

    g = torch.Generator().manual_seed(5)
    nC, D = n * C, n * n + 2 * n
    parts = [torch.randn(r, nC, generator=g).to(src).cuda() for r in (n, n, n * n)]
    bs = [torch.randn(k, generator=g).cuda() for k in (n, n, n * n)]
    al = [torch.randn(1, generator=g).cuda() for _ in range(3)]
    phi = torch.full((D, nC), float("nan"), dtype=dst, device="cuda")
    bias = torch.empty(D, device="cuda")
    alpha = torch.empty(3, device="cuda")
    p = lambda t: t.data_ptr()
    _lib.check("mhc_pack_dynamic_params", _lib.lib.mhc_pack_dynamic_params(
        p(parts[0]), p(parts[1]), p(parts[2]), _lib.dtype_code(parts[0]), p(bs[0]), p(bs[1]), p(bs[2]),
        p(al[0]), p(al[1]), p(al[2]), p(phi), _lib.dtype_code(phi), p(bias), p(alpha), n, C,
        torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(phi, torch.cat(parts).to(dst))
    assert torch.equal(bias, torch.cat(bs))
    assert torch.equal(alpha, torch.cat(al))
