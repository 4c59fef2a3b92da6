#!/usr/bin/env python3
"""Two comparisons behind launch-path decisions of the library, each printed as a table.

  --forward-paths   dynamic-H bf16 layer, forward alone and whole forward+backward step (both as
                    graphs of ten, like bench.py): the two-launch forward (split-K
                    projection, then the fused coefficient + mix kernel) against the one-launch
                    forward (csrc/layer_fwd_onepass.hip), forced through the library's experiment
                    hook mhc_tuning_set(0, 1 | 2).  The library's default takes the one-launch
                    kernel where phi is at most 256 KB; this table is what that rule was read from.
  --vendor-gemm     the three projection products of the layer (P = x phi^T, dxflat = dP phi,
                    dphi = dP^T x) as plain torch.matmul calls in bf16 (hipBLASLt / rocBLAS) at the
                    benchmark shapes: a reference point for the hand-written projection kernels,
                    whose times are in profiles/layer_step_<config>.txt.

    python mhc.cu_amd/benchmarks/bench_paths.py --forward-paths
    python mhc.cu_amd/benchmarks/bench_paths.py --vendor-gemm
"""
from __future__ import annotations

import argparse
import ctypes
import os
import sys

import torch

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..")
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "mhc.cu_amd"))


def _events(fn, reps):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


_GRAPH_STEPS = 10  # steps per graph replay, as in bench.py: a replay costs ~5 us by itself


def _graph(step):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(_GRAPH_STEPS):
            step()
    g.replay()
    torch.cuda.synchronize()
    return g


def forward_paths(reps):
    import bench  # the repository's bench.py: its Step drives the C ABI on device buffers
    from mhc._lib import lib

    lib.mhc_tuning_set.restype = ctypes.c_int
    lib.mhc_tuning_set.argtypes = [ctypes.c_int, ctypes.c_int]
    print("dynamic H, bf16, 20 Sinkhorn iterations; us per call, warm caches")
    print("%5s %3s %5s %8s | %8s %8s | %9s %9s" % ("B", "n", "C", "phi KB", "fwd two", "fwd one", "step two", "step one"))
    try:
        for n in (4, 3, 2):
            for B in (64, 320, 1280, 4096):
                for C in (512, 1280, 2560, 4096):
                    if B * n * C > 4096 * 4 * 2560:
                        continue
                    step = bench.Step(dict(kind="dynamic", B=B, n=n, C=C, dtype="bf16", bwd=True), "L", torch)
                    r = []
                    for mode in (1, 2):
                        lib.mhc_tuning_set(0, mode)
                        r.append(_events(_graph(step.forward).replay, reps // 2) / _GRAPH_STEPS)
                    for mode in (1, 2):
                        lib.mhc_tuning_set(0, mode)
                        r.append(_events(_graph(step.step).replay, reps // 2) / _GRAPH_STEPS)
                    print("%5d %3d %5d %8.0f | %8.1f %8.1f | %9.1f %9.1f" %
                          (B, n, C, 2 * (n * n + 2 * n) * n * C / 1024, *r), flush=True)
                    del step
    finally:
        lib.mhc_tuning_set(0, 0)


def vendor_gemm(reps):
    print("torch.matmul, bf16 operands and result; us per call, warm caches")
    print("%5s %3s %5s | %12s %14s %14s" % ("B", "n", "C", "P = x phi^T", "dxflat = dP phi", "dphi = dP^T x"))
    for B, n, C in ((320, 4, 1280), (1280, 4, 2560), (256, 8, 1280), (128, 32, 1280)):
        nC, D = n * C, n * n + 2 * n
        x = torch.randn(B, nC, device="cuda", dtype=torch.bfloat16)
        phi = torch.randn(D, nC, device="cuda", dtype=torch.bfloat16)
        dP = torch.randn(B, D, device="cuda", dtype=torch.bfloat16)
        print("%5d %3d %5d | %12.1f %14.1f %14.1f" % (B, n, C, _events(lambda: x @ phi.t(), reps),
                                                     _events(lambda: dP @ phi, reps), _events(lambda: dP.t() @ x, reps)),
              flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--forward-paths", action="store_true")
    ap.add_argument("--vendor-gemm", action="store_true")
    ap.add_argument("--reps", type=int, default=100)
    a = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("bench_paths.py: no GPU visible")
    if a.forward_paths:
        forward_paths(a.reps)
    if a.vendor_gemm:
        vendor_gemm(a.reps)
    if not (a.forward_paths or a.vendor_gemm):
        ap.print_help()


if __name__ == "__main__":
    main()
