"""The Python benchmark harness (mhc.cu_amd/benchmarks/bench_layer.py, the counterpart of the
reference's src/python/benchmarks/bench_layer.py:148-456) runs end to end on one configuration and
prints its four tables: static / dynamic H x forward / forward+backward, fused against a plain
PyTorch layer on the same GPU."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SCRIPT = os.path.join(ROOT, "mhc.cu_amd", "benchmarks", "bench_layer.py")

TITLES = ["Static H Path", "Dynamic H Path", "Backward Pass Static H", "Backward Pass Dynamic H Path"]
ROW = re.compile(r"^\s*(\d+)\s+(\d+)\s+(\d+)\s+([0-9.]+)\s+([0-9.]+)\s+([0-9.]+)x\s*$")


@pytest.mark.gpu
def test_bench_layer_prints_its_four_tables():
    cmd = [sys.executable, SCRIPT, "--batch", "64", "--hidden", "256", "--expansion", "4", "--backward",
           "--warmup", "3", "--runs", "10"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    out = p.stdout
    pos = [out.find(t) for t in TITLES]
    assert all(i >= 0 for i in pos) and pos == sorted(pos), out[-2000:]
    rows = [m.groups() for m in (ROW.match(line) for line in out.splitlines()) if m]
    assert len(rows) == 4, out[-2000:]
    for B, C, n, fused_ms, plain_ms, speedup in rows:
        assert (int(B), int(C), int(n)) == (64, 256, 4)
        assert 0 < float(fused_ms) < 10 and 0 < float(plain_ms) < 100 and float(speedup) > 0
