"""Host-side checks of the C ABI that need no GPU: the library loads, exports every symbol the
header declares, validates arguments before touching the device, and sizes its workspace."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mhc_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"MHC_API\s+[\w\s\*]+?\b(mhc_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from mhc import _lib

    names = _declared_symbols()
    assert len(names) >= 14, names
    for name in names:
        assert hasattr(_lib.lib, name), f"{name} declared in mhc_hip.h but not exported"
        assert name in _lib._SIGNATURES, f"{name} has no ctypes signature in the binding"
    assert _lib.lib.mhc_abi_version() == 2


def test_library_exports_nothing_the_header_does_not_declare():
    """The product library carries no experiment hooks, probes or other undeclared entry points (those
    live in libmhc_hip_tuning.so / libmhc_probe.so)."""
    import subprocess

    from mhc import _lib

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T " in l)
    assert exported == _declared_symbols()


def test_status_strings():
    from mhc import _lib

    seen = set()
    for code in range(0, 9):
        s = _lib.lib.mhc_status_string(code).decode()
        assert s and s != "unknown status"
        seen.add(s)
    assert len(seen) == 9
    assert _lib.lib.mhc_status_string(99).decode() == "unknown status"


def test_workspace_queries():
    from mhc import _lib

    L = _lib.lib
    for (B, n, C) in [(320, 4, 1280), (1280, 4, 2560), (256, 8, 1280), (128, 32, 1280), (1, 1, 8)]:
        d = L.mhc_layer_dynamic_workspace_bytes(B, n, C)
        s = L.mhc_layer_static_workspace_bytes(B, n, C)
        assert d > 0 and d % 256 == 0 and s > 0 and s % 256 == 0
        assert d < 512 * 1024 * 1024
    assert L.mhc_layer_dynamic_workspace_bytes(8, 33, 64) == 0   # n out of range
    assert L.mhc_layer_dynamic_workspace_bytes(0, 4, 64) == 0
    assert L.mhc_rmsnorm_bwd_workspace_bytes(8, 128) > 0
    assert L.mhc_sinkhorn_knopp_bwd_workspace_bytes(1, 200, 4, 5) == 0


def test_argument_validation_happens_before_any_launch():
    """Bad arguments are rejected with distinct codes; nothing is launched, so this runs without a GPU."""
    from mhc import _lib

    L = _lib.lib
    P = ctypes.c_void_p
    buf = (ctypes.c_char * 4096)()
    a = ctypes.addressof(buf)
    a16 = P((a + 255) // 256 * 256)
    odd = P(a16.value + 4)
    fwd = lambda **kw: L.mhc_layer_fwd_dynamic(
        kw.get("x", a16), kw.get("xd", 0), a16, 0, a16, 0, a16, a16, None, kw.get("y", a16), kw.get("yd", 0),
        a16, a16, a16, a16, a16, a16, kw.get("sk", None), kw.get("B", 2), kw.get("n", 4), kw.get("C", 8),
        kw.get("T", 20), 1e-6, kw.get("ws", None), kw.get("wsb", 0), None)
    assert fwd(n=0) == 2 and fwd(n=33) == 2            # MHC_ERR_BAD_N
    assert fwd(B=0) == 3                               # MHC_ERR_BAD_SHAPE
    assert fwd(C=32768 + 8) == 3 and fwd(C=32768) == 6   # MHC_MAX_C
    # no bound on the batch beyond B * n * C <= 2^40 (samples are not tied to a 16-bit grid dimension)
    assert fwd(n=9, B=65536) == 6 and fwd(n=32, B=1 << 20) == 6 and fwd(n=32, B=1 << 30, C=64) == 3
    # iteration counts beyond what the backward keeps in LDS are refused up front, per n
    assert [L.mhc_max_sinkhorn_iters(n) for n in (0, 1, 4, 5, 8, 9, 16, 17, 32, 33)] == \
        [0, 256, 256, 256, 256, 256, 256, 256, 256, 0]
    assert fwd(n=4, T=257) == 3 and fwd(n=8, T=257) == 3 and fwd(n=32, T=257) == 3 and fwd(T=-1) == 3
    assert fwd(n=4, T=256) == 6 and fwd(n=8, T=256) == 6 and fwd(n=16, T=256) == 6   # next check: workspace
    assert fwd(x=None) == 1                            # MHC_ERR_NULL_POINTER
    assert fwd(xd=7) == 4                              # MHC_ERR_BAD_DTYPE
    assert fwd(xd=0, yd=1) == 4                        # fp32 in / bf16 out is not offered
    assert fwd(x=odd) == 5                             # MHC_ERR_MISALIGNED
    assert fwd() == 6                                  # MHC_ERR_WORKSPACE (none given)
    # [B, iters + 1, 2, NP] floats with NP = n rounded up to 4, 8, 16 or 32
    state = L.mhc_layer_sinkhorn_state_floats
    assert [state(3, n, 20) for n in (1, 4, 5, 8, 9, 16, 17, 32)] == [3 * 21 * 2 * k for k in (4, 4, 8, 8, 16, 16, 32, 32)]
    assert state(3, 33, 20) == 0 and state(0, 4, 20) == 0 and state(3, 4, 0) == 3 * 2 * 4 and state(3, 4, -1) == 0
    assert L.mhc_sinkhorn_knopp_fwd(a16, a16, 1, 129, 4, 3, 1e-8, None) == 3
    assert L.mhc_rmsnorm_fwd(None, 0, a16, 0, a16, None, 1, 8, 1e-5, None) == 1


def test_static_scratch_entry_point_checks_its_limit_before_any_launch():
    """The entry point that allocates nothing refuses shapes beyond its static array up front."""
    from mhc import _lib

    L = _lib.lib
    cap = L.mhc_static_scratch_capacity()
    assert cap == 32 << 20
    assert 0 < L.mhc_layer_fwd_dynamic_scratch_bytes(320, 4, 1280) <= cap
    assert L.mhc_layer_fwd_dynamic_scratch_bytes(8, 33, 64) == 0
    big = (4096, 32, 1280)  # 37 MiB of split-K partial sums
    assert L.mhc_layer_fwd_dynamic_scratch_bytes(*big) > cap
    P = ctypes.c_void_p
    buf = (ctypes.c_char * 4096)()
    a16 = P((ctypes.addressof(buf) + 255) // 256 * 256)
    call = lambda B, n, C: L.mhc_layer_fwd_dynamic_static_scratch(
        a16, 1, a16, 1, a16, 1, a16, a16, None, a16, 1, a16, a16, a16, a16, a16, a16, None, B, n, C, 20, 1e-6, None)
    assert call(*big) == 8          # MHC_ERR_SCRATCH_LIMIT
    assert call(0, 4, 64) == 3      # shape checks come first


def test_python_surface_matches_reference_names():
    import mhc

    for name in ("MHCLayer", "sinkhorn_knopp", "rmsnorm", "mhc_layer_fused", "mhc_layer_fused_dynamic"):
        assert hasattr(mhc, name)
    dyn = mhc.MHCLayer(hidden_dim=128, expansion_rate=4)
    assert dyn.use_dynamic_h is True
    p = dict(dyn.named_parameters())
    assert p["rmsnorm_weight"].shape == (128,) and p["rmsnorm_weight"].dtype == torch.bfloat16
    assert p["phi_pre"].shape == (4, 512) and p["phi_post"].shape == (4, 512)
    assert p["phi_res"].shape == (16, 512)
    assert p["b_pre"].shape == (4,) and p["b_res"].shape == (4, 4) and p["alpha_res"].shape == ()
    assert "H_pre" not in p
    sta = mhc.MHCLayer(hidden_dim=128, expansion_rate=4, use_dynamic_h=False)
    p = dict(sta.named_parameters())
    assert set(p) == {"rmsnorm_weight", "H_pre", "H_post", "H_res"}
    assert p["H_res"].shape == (4, 4) and p["H_pre"].dtype == torch.float32


def test_cpu_tensors_are_refused_not_silently_computed():
    """There is no CPU path behind the operators: CPU tensors raise."""
    import mhc

    layer = mhc.MHCLayer(hidden_dim=16, expansion_rate=4, use_dynamic_h=False)
    with pytest.raises(RuntimeError):
        layer(torch.randn(2, 4, 16))


def test_torch_extension_is_built_and_bound_to_the_same_library():
    """The operators run through the compiled PyTorch extension (no Python fallback); it links the same
    libmhc_hip.so that the ctypes handle holds."""
    from mhc import _lib, ops

    ext = ops._ext
    assert ext.__file__.endswith(".so") and "mhc_torch_ext" in ext.__file__
    assert ext.abi_version() == _lib.lib.mhc_abi_version()
    for name in ("mhc_layer_dynamic", "mhc_layer_static", "mhc_layer_inference", "sinkhorn_knopp", "rmsnorm",
                 "set_param_cache"):
        assert hasattr(ext, name)
    with open("/proc/self/maps") as f:
        libs = {line.split()[-1] for line in f if "libmhc_hip" in line}
    assert len(libs) == 1, libs
