"""bench.py's contract with whoever runs it: one JSON line with the agreed keys, one GPU only, byte
counts that follow the closed forms, and profile summaries whose headers name commands that exist."""
import glob
import json
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_bytes_follow_the_closed_forms():
    # c2, layer-level view: forward 2 * (2 BnC) + 2 nC D, backward 2 * (3 BnC) + 2 nC D + 4 nC D
    B, n, C, D = 320, 4, 1280, 24
    fwd, bwd = bench.algorithmic_bytes(bench.CONFIGS["c2"], "L")
    assert fwd == 2 * 2 * B * n * C + 2 * n * C * D == 6799360
    assert bwd == 2 * 3 * B * n * C + 6 * n * C * D == 10567680
    # kernel-level view adds f (forward) and f, df (backward)
    fk, bk = bench.algorithmic_bytes(bench.CONFIGS["c2"], "K")
    assert fk - fwd == 2 * B * C and bk - bwd == 2 * 2 * B * C
    # c1: static fp32 forward only, no phi
    f1, b1 = bench.algorithmic_bytes(bench.CONFIGS["c1"], "L")
    assert (f1, b1) == (2 * 4 * 320 * 4 * 1280, 0)


def test_profiled_constants_cover_every_configuration():
    for c in bench.CONFIGS:
        d = bench.PROFILED_DOMINANT[c]
        assert d["us"] > 0 and d["bytes"] > 0
        frac = d["bytes"] / (d["us"] * 1e-6) / 1e9 / bench.HBM_PEAK_GBS
        assert 0 < frac < 1, (c, frac)
        assert bench.MEASURED_TRAFFIC["bytes"][c] >= sum(bench.algorithmic_bytes(bench.CONFIGS[c], "L")) * 0.99
        assert os.path.exists(os.path.join(ROOT, "profiles", f"layer_step_{c}.txt"))
    assert re.fullmatch(r"[0-9a-f]{7,}", bench.PROFILED_AT) and bench.MEASURED_TRAFFIC["commit"] == bench.PROFILED_AT


def test_profile_summaries_carry_revision_and_runnable_commands():
    files = sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt")))
    assert files
    for path in files:
        head = [l for l in open(path).read().splitlines() if l.startswith("#")]
        text = "\n".join(head)
        assert re.search(r"# revision: [0-9a-f]{7,}", text), path
        assert "command" in text, path
        # every program or script a header names is a committed file (built programs: their source)
        for m in re.finditer(r"(?:python |^#\s+|; |&& )((?:mhc\.cu_amd|tests)/[\w./-]+|bench\.py)", text, flags=re.M):
            name = m.group(1)
            cand = [name, name + ".cpp", name + ".py"]
            assert any(os.path.exists(os.path.join(ROOT, c)) for c in cand), (path, name)
        assert "_work" not in text, path


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_agreed_keys():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "20", "--warmup", "5"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "single_step_graph_us", "cold_us"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 5 and d["higher_is_better"] is False
    assert d["vs_baseline"] is None and d["data"] == "synthetic" and "workload" in d["config"]
    r_ = d["roofline"]
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "cold_us", "cold_frac", "dominant"):
        assert k in r_, k
    assert r_["bound"] == "hbm" and r_["peak"] == 8000.0 and abs(r_["frac"] - r_["achieved"] / r_["peak"]) < 1e-9
    assert 0 < r_["cold_frac"] < r_["frac"] < 1
    assert abs(d["value"] - d["ms_per_step"] * 1e3) < 1e-6
    cb = d["cpu_baseline"]
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in cb, k
    assert cb["kind"] == "port" and cb["cores"] >= 1
    # the box's own read and write rates, for comparing lines from different boxes (None without the probe library)
    assert d["box"] is None or (1000 < d["box"]["write_GBs"] < 8000 and 1000 < d["box"]["read_GBs"] < 8000)
