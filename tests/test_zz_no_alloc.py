"""mhc_layer_fwd_dynamic_static_scratch (the entry point that allocates nothing: its scratch is a
device array inside the library) against mhc_layer_fwd_dynamic on the same inputs, through the
C ABI.  Both run the same kernels, so every output must agree bit for bit.  Two calls in a row
share the array; the second is smaller, so stale contents of the first must not leak into it."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(B, n, C, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    D = n * n + 2 * n
    x = torch.randn(B, n, C, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(C, generator=g)).to(dtype).cuda()
    phi = (0.02 * torch.randn(D, n * C, generator=g)).to(dtype).cuda()
    bias = (0.1 * torch.randn(D, generator=g)).cuda()
    alpha = torch.tensor([0.3, 0.2, 0.5]).cuda()
    return x, w, phi, bias, alpha


def _run(entry, B, n, C, dtype, seed, T=20, eps=1e-6):
    from mhc import _lib
    from mhc._lib import check, dtype_code, lib, ptr

    x, w, phi, bias, alpha = _inputs(B, n, C, dtype, seed)
    D = n * n + 2 * n
    f32 = dict(dtype=torch.float32, device="cuda")
    out = dict(y=torch.empty_like(x), Hp=torch.empty(B, n, **f32), Ho=torch.empty(B, n, **f32),
               M=torch.empty(B, n, n, **f32), P=torch.empty(B, D, **f32), r=torch.empty(B, **f32),
               q=torch.empty(B, **f32), sk=torch.empty(lib.mhc_layer_sinkhorn_state_floats(B, n, T), **f32))
    for t in out.values():
        t.fill_(float("nan"))
    common = (ptr(x), dtype_code(x), ptr(w), dtype_code(w), ptr(phi), dtype_code(phi), ptr(bias), ptr(alpha),
              None, ptr(out["y"]), dtype_code(out["y"]), ptr(out["Hp"]), ptr(out["Ho"]), ptr(out["M"]),
              ptr(out["P"]), ptr(out["r"]), ptr(out["q"]), ptr(out["sk"]), B, n, C, T, eps)
    st = _lib.stream_ptr(x.device)
    if entry == "static_scratch":
        check("mhc_layer_fwd_dynamic_static_scratch", lib.mhc_layer_fwd_dynamic_static_scratch(*common, st))
    else:
        nbytes = lib.mhc_layer_dynamic_workspace_bytes(B, n, C)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        check("mhc_layer_fwd_dynamic", lib.mhc_layer_fwd_dynamic(*common, ptr(ws), ws.numel(), st))
    torch.cuda.synchronize()
    NP = out["sk"].numel() // (B * (T + 1) * 2)  # rows and columns n..NP-1 of the saved state are padding
    out["sk"] = out["sk"].reshape(B, T + 1, 2, NP)[:, :T, :, :n]
    return {k: v.float().cpu() for k, v in out.items()}


@pytest.mark.parametrize("n,C,dtype", [(8, 256, torch.bfloat16), (4, 512, torch.float32),
                                       (16, 128, torch.bfloat16)])
def test_static_scratch_forward_matches_workspace_forward(n, C, dtype):
    from mhc._lib import lib

    assert lib.mhc_static_scratch_init() == 0
    for call, B in enumerate((96, 40)):  # the second call is smaller and reuses the array
        assert 0 < lib.mhc_layer_fwd_dynamic_scratch_bytes(B, n, C) <= lib.mhc_static_scratch_capacity()
        got = _run("static_scratch", B, n, C, dtype, seed=call)
        ref = _run("workspace", B, n, C, dtype, seed=call)
        for k in ref:
            assert torch.isfinite(got[k]).all(), (call, k)
            assert torch.equal(got[k], ref[k]), (call, k, float((got[k] - ref[k]).abs().max()))


def test_static_scratch_forward_allocates_nothing_and_replays_in_a_graph():
    """What the entry point is for: no device memory is taken by a call (free memory is unchanged over
    eager calls once the array's address has been looked up), and after mhc_static_scratch_init() it
    can be captured into a HIP graph; every replay, with unrelated eager work and synchronisations
    between the replays, reproduces the eager result bit for bit."""
    from mhc import _lib
    from mhc._lib import check, dtype_code, lib, ptr

    B, n, C, T, eps, dtype = 64, 8, 256, 20, 1e-6, torch.bfloat16
    x, w, phi, bias, alpha = _inputs(B, n, C, dtype, 5)
    D = n * n + 2 * n
    f32 = dict(dtype=torch.float32, device="cuda")
    out = dict(y=torch.empty_like(x), Hp=torch.empty(B, n, **f32), Ho=torch.empty(B, n, **f32),
               M=torch.empty(B, n, n, **f32), P=torch.empty(B, D, **f32), r=torch.empty(B, **f32),
               q=torch.empty(B, **f32))
    scratch = torch.zeros(1 << 20, device="cuda")  # allocated before the free-memory readings
    assert lib.mhc_static_scratch_init() == 0

    def call():
        st = _lib.stream_ptr(x.device)
        check("mhc_layer_fwd_dynamic_static_scratch",
              lib.mhc_layer_fwd_dynamic_static_scratch(ptr(x), dtype_code(x), ptr(w), dtype_code(w), ptr(phi),
                                                       dtype_code(phi), ptr(bias), ptr(alpha), None, ptr(out["y"]),
                                                       dtype_code(out["y"]), ptr(out["Hp"]), ptr(out["Ho"]), ptr(out["M"]),
                                                       ptr(out["P"]), ptr(out["r"]), ptr(out["q"]), None, B, n, C, T, eps, st))

    call()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "a call through the no-allocation entry point took device memory"
    eager = {k: v.clone() for k, v in out.items()}

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        for t in out.values():
            t.fill_(float("nan"))
        scratch.add_(1.0).sum().item()  # eager work + a host sync between replays
        graph.replay()
        torch.cuda.synchronize()
        for k, v in out.items():
            assert torch.equal(v, eager[k]), (rep, k)


def test_static_scratch_refuses_shapes_beyond_its_array():
    from mhc._lib import lib

    B, n, C = 4096, 32, 1280
    assert lib.mhc_layer_fwd_dynamic_scratch_bytes(B, n, C) > lib.mhc_static_scratch_capacity()
    x, w, phi, bias, alpha = _inputs(2, 4, 64, torch.bfloat16, 0)  # never dereferenced: refused before any launch
    from mhc._lib import ptr
    st = lib.mhc_layer_fwd_dynamic_static_scratch(ptr(x), 1, ptr(w), 1, ptr(phi), 1, ptr(bias), ptr(alpha), None,
                                                  ptr(x), 1, ptr(bias), ptr(bias), ptr(bias), ptr(bias),
                                                  ptr(bias), ptr(bias), None, B, n, C, 20, 1e-6, None)
    assert st == 8
