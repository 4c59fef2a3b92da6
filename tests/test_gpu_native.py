"""Runs the native (no Python in the measured program) parity test of the C ABI.

tests/native/test_mhc_layer is built beforehand (make -C tests/native, or __graft_entry__.build());
it compares every output of the dynamic and static layer calls with the plain-C fp64 oracle at
1e-5 and exits non-zero on any mismatch.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "native", "test_mhc_layer")


@pytest.mark.gpu
def test_native_operator_parity_executable():
    """tests/native/test_ops: mhc_sinkhorn_knopp_* and mhc_rmsnorm_* against the C oracle."""
    exe = os.path.join(HERE, "native", "test_ops")
    assert os.path.exists(exe), "build tests/native first (make -C tests/native)"
    p = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(p.stdout[-4000:])
    assert p.returncode == 0, p.stdout[-4000:] + p.stderr[-2000:]
    assert "all comparisons passed" in p.stdout


@pytest.mark.gpu
def test_native_parity_executable():
    assert os.path.exists(EXE), "build tests/native first (make -C tests/native)"
    p = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    print(p.stdout[-3000:])
    assert p.returncode == 0, p.stdout[-3000:] + p.stderr[-2000:]
    assert "all comparisons passed" in p.stdout
