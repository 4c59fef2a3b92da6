#!/usr/bin/env python3
"""Benchmark of the fused mHC layer path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--mode graph|eager]
                    [--graph-steps G]

A step is one forward + backward pass of the layer over one batch of synthetic, seeded input
that is already resident in HBM, issued through the C ABI (libmhc_hip.so).  Prints ONE JSON
line.  `value` is microseconds per step over K back-to-back steps (wall clock, synchronised on
both sides; in graph mode the K steps are K / G replays of a HIP graph that holds G steps, the
rest as single-step replays); `roofline` prices the same step's device time (HIP events on the launch stream)
against the algorithmic HBM bytes of the configuration; `cpu_baseline` is the naive PyTorch
restatement of the layer (the oracle) timed on this machine's host cores.

Configurations (BASELINE.json order): c1 static fp32 forward; c2..c5 dynamic bf16 fwd+bwd.
View "L" (default): the layer computes f = RMSNorm(x_agg) * w itself, as MHCLayer does.
View "K": f [B, C] is an input and df an output (kernel-level view of the configurations).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "mhc.cu_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes of one step (all launches, graph-less run), from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE summed over the step's kernels and scaled by what the same counters read for
# `--copy-calibration` (a 64 MiB copy).  Filled from the committed counter summary
# (profiles/hbm_traffic_counters.txt); `commit` is the revision of the kernels the counters ran on.
MEASURED_TRAFFIC = {
    "commit": "44e4d8b",
    "bytes": {"c1": 13281066, "c2": 37946871, "c3": 246954758, "c4": 64736245, "c5": 577687318},
}

# The kernel with the largest share of a step's device time, from the committed kernel-trace summaries
# (profiles/layer_step_<config>.txt): average duration per dispatch and the HBM bytes the algorithm
# needs that kernel to move (its own inputs and outputs once; for the split projections the partial
# sums are not counted).
PROFILED_AT = "44e4d8b"
PROFILED_DOMINANT = {
    "c1": dict(kernel="layer_fwd_small_kernel<float,float,4,4,2>", us=6.60, bytes=2 * 4 * 320 * 4 * 1280),
    # sample-resident backward kernel: reads dy and x, writes the partial dx and the fp32 rows the batch sums are made of
    "c2": dict(kernel="bwd_resident_kernel<4,bf16 w,2 items,5 tile waves>", us=10.07, bytes=3 * 2 * 320 * 4 * 1280 + 4 * 320 * 1280),
    "c3": dict(kernel="bwd_slab_kernel<bf16>", us=24.35, bytes=3 * 2 * 1280 * 4 * 2560 + 2 * 24 * 10240 + 4 * 24 * 10240),
    "c4": dict(kernel="bwd_resident_kernel<8,bf16 w,1 item,10 tile waves>", us=11.94, bytes=3 * 2 * 256 * 8 * 1280 + 4 * 256 * 1280),
    "c5": dict(kernel="dphi_large_kernel<9,true>", us=35.90, bytes=2 * 128 * 40960 + 4 * 1088 * 40960),
}

CONFIGS = {
    "c1": dict(kind="static", B=320, n=4, C=1280, dtype="f32", bwd=False),
    "c2": dict(kind="dynamic", B=320, n=4, C=1280, dtype="bf16", bwd=True),
    "c3": dict(kind="dynamic", B=1280, n=4, C=2560, dtype="bf16", bwd=True),
    "c4": dict(kind="dynamic", B=256, n=8, C=1280, dtype="bf16", bwd=True),
    "c5": dict(kind="dynamic", B=128, n=32, C=1280, dtype="bf16", bwd=True),
}
T_ITERS, EPS = 20, 1e-6


def algorithmic_bytes(cfg, view):
    """Compulsory HBM traffic of one step: (forward, backward) bytes.

    forward : read x [+ f], read phi (dynamic), write y
    backward: read dy, x [+ f], read phi, write dx [+ df], write dphi (fp32)
    """
    B, n, C = cfg["B"], cfg["n"], cfg["C"]
    s = 4 if cfg["dtype"] == "f32" else 2
    BnC, BC, nC, D = B * n * C, B * C, n * C, n * n + 2 * n
    fvec = BC if view == "K" else 0
    phi = 2 * nC * D if cfg["kind"] == "dynamic" else 0
    fwd = s * (BnC + fvec) + phi + s * BnC
    bwd = 0
    if cfg["bwd"]:
        bwd = s * (2 * BnC + fvec) + phi + s * (BnC + fvec) + 2 * phi  # dphi fp32 = 2x bf16 phi bytes
    return fwd, bwd


def kernels_changed_since(commit):
    """True if the kernel sources differ from the revision a committed profile ran on, False if they do not,
    None where that cannot be told (no git checkout, as on a box that only holds a copy of the tree)."""
    import subprocess
    if not os.path.isdir(os.path.join(ROOT, ".git")):
        return None
    try:
        rc = subprocess.run(["git", "-C", ROOT, "diff", "--quiet", commit, "HEAD", "--", "mhc.cu_amd/csrc"],
                            stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=20).returncode
    except (OSError, subprocess.SubprocessError):
        return None
    return {0: False, 1: True}.get(rc)


def dominant_kernel(config):
    """roofline.dominant: the step's largest kernel as profiled (not re-timed here: HIP events see whole
    entry points, not the launches inside them); `profiled_at` is the revision the profile ran on."""
    d = dict(PROFILED_DOMINANT[config])
    d["frac"] = d["bytes"] / (d["us"] * 1e-6) / 1e9 / HBM_PEAK_GBS
    d["source"] = f"profiles/layer_step_{config}.txt"
    d["profiled_at"] = PROFILED_AT
    d["kernels_changed_since"] = kernels_changed_since(PROFILED_AT)
    if d["kernels_changed_since"]:
        print(f"bench.py: csrc/ has changed since {PROFILED_AT}, the revision roofline.dominant and roofline.traffic "
              "were profiled at; regenerate profiles/ and the constants at the top of this file", file=sys.stderr)
    return d


def synthetic_inputs(torch, cfg, with_f):
    """Seeded synthetic inputs of a configuration, on the host, as fp32 tensors: x, dy (and f) ~ N(0,1)
    from seed 0; parameters from seed 1: phi ~ N(0, 0.02^2), bias = 0, alpha = 0.01, w = 1 (dynamic),
    logits ~ N(0,1) (static).  For the bf16 configurations everything stored in bf16 on the device is
    rounded to bf16 here, so the CPU baseline sees the same values as the GPU."""
    B, n, C = cfg["B"], cfg["n"], cfg["C"]
    gd, gp = torch.Generator().manual_seed(0), torch.Generator().manual_seed(1)
    x = torch.randn(B, n, C, generator=gd)
    dy = torch.randn(B, n, C, generator=gd)
    f = torch.randn(B, C, generator=gd) if with_f else None
    if cfg["kind"] == "dynamic":
        nC = n * C
        p = {"w": torch.ones(C),
             "phi_pre": torch.randn(n, nC, generator=gp) * 0.02,
             "phi_post": torch.randn(n, nC, generator=gp) * 0.02,
             "phi_res": torch.randn(n * n, nC, generator=gp) * 0.02,
             "alpha_pre": torch.tensor(0.01), "alpha_post": torch.tensor(0.01), "alpha_res": torch.tensor(0.01),
             "b_pre": torch.zeros(n), "b_post": torch.zeros(n), "b_res": torch.zeros(n, n)}
    else:
        p = {"w": torch.ones(C), "H_pre": torch.randn(n, generator=gp), "H_post": torch.randn(n, generator=gp),
             "H_res": torch.randn(n, n, generator=gp)}
    if cfg["dtype"] == "bf16":
        rb = lambda t: t.bfloat16().float()
        x, dy = rb(x), rb(dy)
        f = None if f is None else rb(f)
        for k in ("w", "phi_pre", "phi_post", "phi_res"):
            if k in p:
                p[k] = rb(p[k])
    return x, dy, f, p


class Step:
    """Pre-allocated tensors and the two C-ABI calls of one configuration."""

    def __init__(self, cfg, view, torch, lib=None):
        from mhc import _lib

        self.torch, self.lib, self._lib = torch, (lib if lib is not None else _lib.lib), _lib
        self.cfg, self.view = cfg, view
        B, n, C = cfg["B"], cfg["n"], cfg["C"]
        dev = torch.device("cuda:0")
        act = torch.float32 if cfg["dtype"] == "f32" else torch.bfloat16
        bf = cfg["dtype"] == "bf16"
        self.dynamic = cfg["kind"] == "dynamic"
        x, dy, f, p = synthetic_inputs(torch, cfg, with_f=(view == "K"))
        self.host = dict(x=x, dy=dy, f=f, p=p)
        to = lambda t, dt: t.to(dt).to(dev).contiguous()
        self.x, self.dy = to(x, act), to(dy, act)
        self.f = None if f is None else to(f, act)
        self.w = to(p["w"], torch.bfloat16 if bf else torch.float32)
        D = n * n + 2 * n
        f32 = dict(dtype=torch.float32, device=dev)
        self.y = torch.empty((B, n, C), dtype=act, device=dev)
        self.dx = torch.empty_like(self.x)
        self.df = None if f is None else torch.empty_like(self.f)
        self.dw = torch.empty(C, **f32)
        self.q = torch.empty(B, **f32)
        if self.dynamic:
            phi = torch.cat([p["phi_pre"], p["phi_post"], p["phi_res"]], 0)
            self.phi = to(phi, torch.bfloat16 if bf else torch.float32)
            self.bias = to(torch.cat([p["b_pre"], p["b_post"], p["b_res"].reshape(-1)]), torch.float32)
            self.alpha = to(torch.stack([p["alpha_pre"], p["alpha_post"], p["alpha_res"]]), torch.float32)
            self.Hp, self.Ho = torch.empty((B, n), **f32), torch.empty((B, n), **f32)
            self.M, self.P = torch.empty((B, n, n), **f32), torch.empty((B, D), **f32)
            self.r = torch.empty(B, **f32)
            self.sk = torch.empty(max(self.lib.mhc_layer_sinkhorn_state_floats(B, n, T_ITERS), 1), **f32)
            self.dphi = torch.empty((D, n * C), **f32)
            self.dbias, self.dalpha = torch.empty(D, **f32), torch.empty(3, **f32)
            nbytes = self.lib.mhc_layer_dynamic_workspace_bytes(B, n, C)
        else:
            self.Hl = [to(p[k], torch.float32) for k in ("H_pre", "H_post", "H_res")]
            self.Hp, self.Ho = torch.empty(n, **f32), torch.empty(n, **f32)
            self.M = torch.empty((n, n), **f32)
            self.dH = [torch.empty(n, **f32), torch.empty(n, **f32), torch.empty((n, n), **f32)]
            nbytes = self.lib.mhc_layer_static_workspace_bytes(B, n, C)
        self.ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)

    def _stream(self):
        return ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def forward(self):
        L, c, p, dc = self.lib, self.cfg, self._lib.ptr, self._lib.dtype_code
        B, n, C = c["B"], c["n"], c["C"]
        if self.dynamic:
            st = L.mhc_layer_fwd_dynamic(p(self.x), dc(self.x), p(self.w), dc(self.w), p(self.phi), dc(self.phi),
                                         p(self.bias), p(self.alpha), p(self.f), p(self.y), dc(self.y),
                                         p(self.Hp), p(self.Ho), p(self.M), p(self.P), p(self.r), p(self.q),
                                         p(self.sk), B, n, C, T_ITERS, EPS, p(self.ws), self.ws.numel(),
                                         self._stream())
        else:
            st = L.mhc_layer_fwd(p(self.x), dc(self.x), p(self.w), dc(self.w), p(self.Hl[0]), p(self.Hl[1]),
                                 p(self.Hl[2]), p(self.f), p(self.y), dc(self.y), p(self.Hp), p(self.Ho),
                                 p(self.M), p(self.q), B, n, C, T_ITERS, EPS, p(self.ws), self.ws.numel(),
                                 self._stream())
        self._lib.check("forward", st)

    def backward(self):
        L, c, p, dc = self.lib, self.cfg, self._lib.ptr, self._lib.dtype_code
        B, n, C = c["B"], c["n"], c["C"]
        if self.dynamic:
            st = L.mhc_layer_bwd_dynamic(p(self.dy), dc(self.dy), p(self.x), dc(self.x), p(self.w), dc(self.w),
                                         p(self.phi), dc(self.phi), p(self.bias), p(self.alpha), p(self.f),
                                         p(self.Hp), p(self.Ho), p(self.M), p(self.P), p(self.r), p(self.q),
                                         p(self.sk), p(self.dx), p(self.df), p(self.dw), p(self.dphi), p(self.dbias),
                                         p(self.dalpha), B, n, C, T_ITERS, EPS, p(self.ws), self.ws.numel(),
                                         self._stream())
        else:
            st = L.mhc_layer_bwd(p(self.dy), dc(self.dy), p(self.x), dc(self.x), p(self.w), dc(self.w),
                                 p(self.Hl[0]), p(self.Hl[1]), p(self.Hl[2]), p(self.f), p(self.Hp), p(self.Ho),
                                 p(self.M), p(self.q), p(self.dx), p(self.df), p(self.dw), p(self.dH[0]),
                                 p(self.dH[1]), p(self.dH[2]), B, n, C, T_ITERS, EPS, p(self.ws),
                                 self.ws.numel(), self._stream())
        self._lib.check("backward", st)

    def step(self):
        self.forward()
        if self.cfg["bwd"]:
            self.backward()


def trimmed_mean(v):
    v = sorted(v)
    k = len(v) // 10
    v = v[k:len(v) - k] if len(v) > 2 * k else v
    return sum(v) / len(v)


def event_times(torch, fn, reps, flush=None):
    """Device time of fn() in microseconds, one HIP-event pair per call on the current stream
    (used for the cold-cache figure; an event pair alone costs several microseconds here)."""
    out = []
    for _ in range(reps):
        if flush is not None:
            flush.fill_(1.0)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        out.append(e0.elapsed_time(e1) * 1e3)
    return out


def event_time_batched(torch, fn, reps, rounds=5):
    """Average device time of fn() in microseconds: `reps` back-to-back calls between ONE event
    pair on the launch stream (the pair's own overhead is amortised), best of `rounds`."""
    best = float("inf")
    for _ in range(rounds):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        e1.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / reps)
    return best


def physical_cores():
    """Physical cores this process may use: distinct (package, core) pairs of the CPUs in its affinity
    mask, capped by the container's CPU quota where one is set."""
    try:
        allowed = sorted(os.sched_getaffinity(0))
    except AttributeError:
        allowed = list(range(os.cpu_count() or 1))
    seen = set()
    for c in allowed:
        try:
            with open(f"/sys/devices/system/cpu/cpu{c}/topology/core_id") as f1, \
                    open(f"/sys/devices/system/cpu/cpu{c}/topology/physical_package_id") as f2:
                seen.add((f2.read().strip(), f1.read().strip()))
        except OSError:
            seen.add(("?", str(c)))
    cores = max(1, len(seen))
    try:
        with open("/sys/fs/cgroup/cpu.max") as f:
            quota, period = f.read().split()
        if quota != "max":
            cores = max(1, min(cores, int(int(quota) / int(period))))
    except (OSError, ValueError):
        pass
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        cores = max(1, min(cores, int(env)))
    return cores


def cpu_baseline(step, torch, budget_s=20.0):
    """The oracle (naive PyTorch layer) on the host cores: same seeded inputs, fp32."""
    from oracle import naive_mhc as nm

    cfg, h = step.cfg, step.host
    cores = physical_cores()
    torch.set_num_threads(cores)
    f = h["f"]

    def run():
        if cfg["kind"] == "dynamic":
            if cfg["bwd"]:
                nm.mhc_dynamic_fwd_bwd(h["x"], h["p"], h["dy"], T_ITERS, EPS, f_inject=f)
            else:
                with torch.no_grad():
                    p = h["p"]
                    nm.mhc_dynamic_forward(h["x"], p["w"], p["phi_pre"], p["phi_post"], p["phi_res"],
                                           p["alpha_pre"], p["alpha_post"], p["alpha_res"], p["b_pre"],
                                           p["b_post"], p["b_res"], T_ITERS, EPS, f_inject=f)
        else:
            if cfg["bwd"]:
                nm.mhc_static_fwd_bwd(h["x"], h["p"], h["dy"], T_ITERS, EPS, f_inject=f)
            else:
                with torch.no_grad():
                    p = h["p"]
                    nm.mhc_static_forward(h["x"], p["w"], p["H_pre"], p["H_post"], p["H_res"], T_ITERS,
                                          EPS, f_inject=f)

    for _ in range(3):
        run()
    times, t_start = [], time.perf_counter()
    while len(times) < 10 or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > 3 * budget_s:
            break
    times.sort()
    med = times[len(times) // 2]
    par = [l.strip() for l in torch.__config__.parallel_info().splitlines()
           if any(k in l for k in ("ATen parallel backend", "OpenMP", "omp_get_max_threads", "MKL", "mkl_get_max_threads"))]
    return {"value": med * 1e6, "unit": "us/layer", "cores": cores, "kind": "port",
            "threads": torch.get_num_threads(), "parallel_info": "; ".join(par)[:400],
            "sample": f"{len(times)} runs of the full {cfg['kind']} "
                      f"{'fwd+bwd' if cfg['bwd'] else 'fwd'} step at B={cfg['B']} n={cfg['n']} C={cfg['C']}, "
                      f"fp32 naive PyTorch layer, median"}


def box_rates(torch):
    """What this box's memory does for plain hand-written kernels (libmhc_probe.so): one 256 MiB buffer read
    and one written, cold, median of 5.  Boxes of the pool differ by 10-20 % in the write rate, which
    moves the write-bound kernels (the 178 MB of dphi at n = 32) by as much; the figures let two bench
    lines from different boxes be compared.  None when the probe library is not built."""
    path = os.path.join(ROOT, "mhc.cu_amd", "mhc", "libmhc_probe.so")
    if not os.path.exists(path):
        return None
    fn = ctypes.CDLL(path).mhc_stream_probe
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                   ctypes.c_void_p]
    nbytes = 256 * 1024 * 1024
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    flush = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.float32, device="cuda")
    src = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for mode, name in ((0, "read_GBs"), (2, "write_GBs")):
        times = []
        for it in range(7):
            flush.fill_(1.0)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            if fn(mode, src.data_ptr(), dst.data_ptr(), nbytes, 16384, sink.data_ptr(), stream) != 0:
                return None
            e1.record()
            e1.synchronize()
            if it >= 2:
                times.append(e0.elapsed_time(e1) * 1e-3)
        times.sort()
        out[name] = round(nbytes / times[len(times) // 2] / 1e9, 1)
    out["protocol"] = "256 MiB, 16-byte nontemporal accesses, 16384 workgroups, cold (512 MiB fill before each), median of 5"
    return out


def stream_probe(torch):
    """Read-only / copy / write-only streaming rates of hand-written kernels and the cost of an empty launch
    (csrc/stream_probe.hip, built into its own libmhc_probe.so)."""
    path = os.path.join(ROOT, "mhc.cu_amd", "mhc", "libmhc_probe.so")
    if not os.path.exists(path):
        raise SystemExit(f"{path} not found: python mhc.cu_amd/build.py")
    fn = ctypes.CDLL(path).mhc_stream_probe
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                   ctypes.c_void_p]
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    flush = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.float32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rows = []
    for mib, cold in ((32, False), (32, True), (128, True), (512, True), (2048, True)):
        nbytes = mib * 1024 * 1024
        src = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for mode, name, moved in ((0, "read", nbytes), (1, "copy", 2 * nbytes), (2, "write", nbytes),
                                  (3, "read", nbytes), (4, "copy", 2 * nbytes), (5, "write", nbytes)):
            for blocks in (2048, 4096, 16384, 65536, 131072):  # few persistent workgroups .. one pass of short ones
                def run():
                    st = fn(mode, src.data_ptr(), dst.data_ptr(), nbytes, blocks, sink.data_ptr(), stream)
                    assert st == 0, st
                for _ in range(3):
                    run()
                times = []
                for _ in range(10):
                    if cold:
                        flush.fill_(1.0)  # the buffers leave the 256 MB Infinity Cache
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    run()
                    e1.record()
                    e1.synchronize()
                    times.append(e0.elapsed_time(e1) * 1e-3)
                times.sort()
                t = times[len(times) // 2]
                rows.append({"kernel": name, "hint": "nt" if mode < 3 else "plain", "MiB": mib,
                             "cache": "cold" if cold else "warm", "blocks": blocks,
                             "us": round(t * 1e6, 1), "GB/s": round(moved / t / 1e9, 1)})
        del src, dst
    # launch floor: a chain of dependent kernels that do nothing, eager and as one HIP graph
    floor = {}
    for blocks in (256, 2048):
        def chain(k=10):
            cur = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)  # the capture stream under capture
            for _ in range(k):
                assert fn(6, None, None, 0, blocks, sink.data_ptr(), cur) == 0
        chain()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            chain()
        for name, run in (("eager", chain), ("graph", g.replay)):
            run()
            best_t = float("inf")
            for _ in range(10):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(10):
                    run()
                e1.record()
                e1.synchronize()
                best_t = min(best_t, e0.elapsed_time(e1) * 1e3 / 100)
            floor[f"{name}_{blocks}_workgroups"] = round(best_t, 2)
    best = {}
    for r in rows:
        key = (r["kernel"], r["MiB"], r["cache"])
        if key not in best or r["GB/s"] > best[key]["GB/s"]:
            best[key] = r
    print(json.dumps({"stream_probe": True, "protocol": "cold: 512 MiB fill before every timed launch; warm: back to back; median of 10, "
                      "HIP events on the launch stream", "rows": rows,
                      "empty_kernel_us_per_launch": floor, "ceiling_GBs": {f"{k[0]}_{k[1]}MiB_{k[2]}": round(v["GB/s"], 1) for k, v in sorted(best.items())}}))


def vendor_gemm(torch, reps=100):
    """torch.matmul on P = x phi^T, dxflat = dP phi and dphi = dP^T x (bf16 operands and result) at the shapes of
    the dynamic configurations; us per call, warm caches, HIP events."""
    rows = []
    for name in ("c2", "c3", "c4", "c5"):
        B, n, C = (CONFIGS[name][k] for k in ("B", "n", "C"))
        nC, D = n * C, n * n + 2 * n
        x = torch.randn(B, nC, device="cuda", dtype=torch.bfloat16)
        phi = torch.randn(D, nC, device="cuda", dtype=torch.bfloat16)
        dP = torch.randn(B, D, device="cuda", dtype=torch.bfloat16)
        rows.append({"config": name, "B": B, "n": n, "C": C,
                     "P=x.phi^T_us": round(event_time_batched(torch, lambda: x @ phi.t(), reps), 1),
                     "dxflat=dP.phi_us": round(event_time_batched(torch, lambda: dP @ phi, reps), 1),
                     "dphi=dP^T.x_us": round(event_time_batched(torch, lambda: dP.t() @ x, reps), 1)})
        print(rows[-1], file=sys.stderr, flush=True)
    print(json.dumps({"vendor_gemm": True, "library": "torch.matmul (hipBLASLt / rocBLAS)", "dtype": "bf16", "rows": rows}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--shape", default=None, metavar="B,n,C",
                    help="a dynamic-H bf16 forward+backward step of another shape than the named configurations "
                         "(for the tables behind the library's path choices); the line then carries no profiled "
                         "constants (roofline.traffic, roofline.dominant)")
    ap.add_argument("--view", default="L", choices=["L", "K"])
    ap.add_argument("--mode", default="graph", choices=["graph", "eager"])
    ap.add_argument("--graph-steps", type=int, default=10,
                    help="steps captured into one HIP graph (a replay costs ~5 us by itself); 1 = one step per replay")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--stream-probe", action="store_true",
                    help="run the library's plain streaming kernels (read-only, copy, write-only; 16-byte accesses, "
                         "all CUs) over 128 MiB .. 2 GiB and print what this GPU delivers to each, HIP events on the "
                         "launch stream: the measured ceiling that the memory-bound kernels are compared with")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="time torch.matmul (the vendor BLAS) on the three projection products of every configuration: "
                         "the reference point for the hand-written projection kernels, not part of the layer path")
    ap.add_argument("--tuning", action="append", default=[], metavar="KEY=VALUE",
                    help="run the step through the tuning build of the library (libmhc_hip_tuning.so, build.py --tuning) "
                         "with one of its path-selection hooks set, e.g. 0=1 / 0=2 = two-launch / one-launch forward, "
                         "7=1 / 7=2 = tiled / two-launch backward for n <= 8 (csrc/tuning.h lists the keys); the line "
                         "then carries the setting and is not the library's default")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run a plain 64 MiB device copy instead of the layer (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters of rocprofv3 --pmc)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 "
              "(every sample is independent: the path shards over the batch)", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if a.stream_probe:
        stream_probe(torch)
        return
    if a.copy_calibration:
        nbytes = 64 * 1024 * 1024
        src = torch.arange(nbytes // 4, dtype=torch.int32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(max(a.steps, 1)):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": True, "bytes_read": nbytes, "bytes_written": nbytes,
                          "copies": max(a.steps, 1)}))
        return
    if a.vendor_gemm:
        vendor_gemm(torch)
        return
    cfg = CONFIGS[a.config]
    if a.shape:
        B_, n_, C_ = (int(t) for t in a.shape.split(","))
        cfg = dict(kind="dynamic", B=B_, n=n_, C=C_, dtype="bf16", bwd=True)
        a.config = f"shape {a.shape}"
    tuned = None
    if a.tuning:
        from mhc import _lib
        tuned = _lib.tuning_lib()
        for kv in a.tuning:
            key, value = (int(t) for t in kv.split("="))
            if tuned.mhc_tuning_set(key, value) != 0:
                sys.exit(f"bench.py: the tuning build refused --tuning {kv}")
    step = Step(cfg, a.view, torch, lib=tuned)

    # ---- warm-up, optional graph capture ---------------------------------------------------
    # A HIP graph replay costs ~5 us on top of its kernels (measured: c2 37.1 us per step with one
    # step per graph, 32.9 with five, 32.4 with ten, 32.1 with twenty; 32.5 for an eager chain that
    # the host keeps fed), so the timed region replays a graph that holds `--graph-steps` steps, the
    # way the layer sits among many others inside a captured model; the figure for one step per
    # replay is reported next to it (roofline.single_step_graph_us).
    for _ in range(max(a.warmup, 1)):
        step.step()
    torch.cuda.synchronize()
    mode, graph, graph1 = a.mode, None, None
    G = max(1, min(a.graph_steps, a.steps))

    def capture(count):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step.step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(count):
                step.step()
        return g

    if mode == "graph":
        try:
            graph1 = capture(1)
            graph = capture(G) if G > 1 else graph1
            for _ in range(max(a.warmup // G, 2)):  # the untimed warm-up runs what the timed region runs
                graph.replay()
            graph1.replay()
            torch.cuda.synchronize()
        except Exception as exc:  # capture is an optimisation of the launch path only
            print(f"bench.py: graph capture failed ({exc}); using eager launches", file=sys.stderr)
            mode, graph, graph1, G = "eager", None, None, 1
    else:
        G = 1
    run1 = graph1.replay if graph1 is not None else step.step

    # ---- timed region: exactly K steps -------------------------------------------------------
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if graph is not None:
        for _ in range(a.steps // G):
            graph.replay()
        for _ in range(a.steps % G):
            graph1.replay()
    else:
        for _ in range(a.steps):
            step.step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    us_per_step = wall / a.steps * 1e6

    # ---- device time with HIP events on the launch stream (warm and cold caches) -------------
    reps = min(max(a.steps, 20), 200)
    if graph is not None:
        dev_step = event_time_batched(torch, graph.replay, max(reps // G, 5)) / G
    else:
        dev_step = event_time_batched(torch, step.step, reps)
    dev_single = event_time_batched(torch, run1, reps) if graph1 is not None else None
    dev_fwd = event_time_batched(torch, step.forward, reps)
    dev_bwd = event_time_batched(torch, step.backward, reps) if cfg["bwd"] else 0.0
    flush = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.float32, device="cuda")
    cold_step = trimmed_mean(event_times(torch, run1, min(reps, 50), flush=flush))
    del flush

    fwd_b, bwd_b = algorithmic_bytes(cfg, a.view)
    alg = fwd_b + bwd_b
    achieved = alg / (dev_step * 1e-6) / 1e9
    out = {
        "metric": "mHC fwd+bwd us/layer" if cfg["bwd"] else "mHC fwd us/layer",
        "value": us_per_step,
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": us_per_step / 1e3,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": f"{a.config}: {cfg['kind']}-H mHC layer "
                               f"{'fwd+bwd' if cfg['bwd'] else 'fwd'} B={cfg['B']} C={cfg['C']} n={cfg['n']} "
                               f"{cfg['dtype']} T={T_ITERS} eps={EPS}",
                   "view": a.view,
                   "launch": (f"graph, {G} steps per replay" if mode == "graph" else mode),
                   "cache": "warm (back-to-back steps)"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC["bytes"].get(a.config) if a.view == "L" else None,
                     "traffic_profiled_at": MEASURED_TRAFFIC["commit"],
                     # the same step with a 512 MiB fill before every one (nothing served from the caches)
                     "cold_us": cold_step, "cold_frac": alg / (cold_step * 1e-6) / 1e9 / HBM_PEAK_GBS,
                     "dominant": dominant_kernel(a.config) if a.config in CONFIGS else None,
                     "kernel": "whole step (all launches of one forward+backward)",
                     "algorithmic_bytes": alg, "device_us": dev_step, "single_step_graph_us": dev_single,
                     "fwd": {"algorithmic_bytes": fwd_b, "device_us": dev_fwd,
                             "achieved": fwd_b / (dev_fwd * 1e-6) / 1e9},
                     "bwd": ({"algorithmic_bytes": bwd_b, "device_us": dev_bwd,
                              "achieved": bwd_b / (dev_bwd * 1e-6) / 1e9} if cfg["bwd"] else None),
                     "cold_cache": {"device_us": cold_step, "achieved": alg / (cold_step * 1e-6) / 1e9,
                                    "flush": "512 MiB fill before every step"}},
    }
    # the three protocols side by side at top level: `value` above (warm, G steps per graph replay), one
    # step per replay (warm), and cold (one step per replay behind a 512 MiB fill)
    out["single_step_graph_us"] = dev_single
    if a.tuning:
        out["config"]["tuning"] = a.tuning
    out["cold_us"] = cold_step
    out["box"] = box_rates(torch)
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(step, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
