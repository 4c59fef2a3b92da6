#!/usr/bin/env python3
"""Layer-level benchmark tables: fused MHCLayer against a plain PyTorch layer on the same GPU.

Counterpart of the reference's src/python/benchmarks/bench_layer.py:148-456: the same command
line, the same nine (batch, hidden, n) configurations (paper appendix A.1), the same four tables
(static / dynamic H, forward / forward+backward), the same protocol (warm-up, a cache flush
before every timed run, one event pair per run, 10 % trimmed mean), so the output can be laid
next to the reference's README tables.  Both layers are fed float32 activations, as there.
--compute selects what the fused layer does with them: "bf16" (default) casts to bfloat16 inside
the layer like the reference's fused kernels do, "fp32" runs the exact float32 kernels, and
"bf16-io" feeds bfloat16 activations and returns bfloat16 (2 bytes per element end to end).

    python mhc.cu_amd/benchmarks/bench_layer.py --all-configs --backward
"""
from __future__ import annotations

import argparse
import os
import sys

import torch
import torch.nn as nn

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))


# ---------------------------------------------------------------------------------------------
# Baseline: the layer written with stock PyTorch operators (what a user would have without the
# fused kernels).  Semantics as in the paper: H_pre = sigmoid, H_post = 2 sigmoid,
# H_res = Sinkhorn-Knopp(exp(.)) with eps added to every denominator.
# ---------------------------------------------------------------------------------------------
def _sinkhorn(logits, iters, eps):
    m = torch.exp(logits)
    for _ in range(iters):
        m = m / (m.sum(dim=-1, keepdim=True) + eps)
        m = m / (m.sum(dim=-2, keepdim=True) + eps)
    return m


def _rms_scale(v, eps):
    return torch.rsqrt(v.pow(2).mean(dim=-1, keepdim=True) + eps)


class PlainStaticLayer(nn.Module):
    def __init__(self, hidden_dim, expansion_rate=4, sinkhorn_iters=20, eps=1e-5, alpha_init=0.01):
        super().__init__()
        n = expansion_rate
        self.iters, self.eps = sinkhorn_iters, eps
        self.rmsnorm_weight = nn.Parameter(torch.ones(hidden_dim))
        self.H_pre = nn.Parameter(torch.zeros(n))
        self.H_post = nn.Parameter(torch.zeros(n))
        self.H_res = nn.Parameter(alpha_init * torch.randn(n, n))

    def forward(self, x):
        h_pre, h_post = torch.sigmoid(self.H_pre), 2.0 * torch.sigmoid(self.H_post)
        m = _sinkhorn(self.H_res, self.iters, self.eps)
        agg = torch.einsum("i,bic->bc", h_pre, x)
        f = agg * _rms_scale(agg, self.eps) * self.rmsnorm_weight
        return torch.einsum("ij,bjc->bic", m, x) + h_post[None, :, None] * f[:, None, :]


class PlainDynamicLayer(nn.Module):
    def __init__(self, hidden_dim, expansion_rate=4, sinkhorn_iters=20, eps=1e-5, alpha_init=0.01):
        super().__init__()
        n, nC = expansion_rate, expansion_rate * hidden_dim
        self.n, self.iters, self.eps = n, sinkhorn_iters, eps
        self.rmsnorm_weight = nn.Parameter(torch.ones(hidden_dim))
        self.phi = nn.Parameter(torch.randn(nC, n * n + 2 * n) * 0.02)
        self.bias = nn.Parameter(torch.zeros(n * n + 2 * n))
        self.alpha = nn.Parameter(torch.full((3,), alpha_init))

    def forward(self, x):
        B, n, C = x.shape
        flat = x.reshape(B, n * C)
        p = (flat * _rms_scale(flat, self.eps)) @ self.phi
        scale = torch.cat([self.alpha[0].expand(n), self.alpha[1].expand(n), self.alpha[2].expand(n * n)])
        t = p * scale + self.bias
        h_pre, h_post = torch.sigmoid(t[:, :n]), 2.0 * torch.sigmoid(t[:, n:2 * n])
        m = _sinkhorn(t[:, 2 * n:].reshape(B, n, n), self.iters, self.eps)
        agg = torch.einsum("bi,bic->bc", h_pre, x)
        f = agg * _rms_scale(agg, self.eps) * self.rmsnorm_weight
        return torch.bmm(m, x) + h_post[:, :, None] * f[:, None, :]


# ---------------------------------------------------------------------------------------------
class CacheFlusher:
    """Overwrites 512 MiB before every timed run (Infinity Cache is 256 MB)."""

    def __init__(self, device):
        self.buf = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.float32, device=device)

    def clear(self):
        self.buf.fill_(1.0)


def _trimmed_mean(times):
    times = sorted(times)
    trim = len(times) // 10
    if trim > 0:
        times = times[trim:-trim]
    return sum(times) / len(times)


def benchmark_forward(layer, B, n, C, device, flusher, warmup, runs, dtype):
    layer.eval()
    times = []
    with torch.no_grad():
        for it in range(warmup + runs):
            x = torch.randn(B, n, C, device=device, dtype=torch.float32).to(dtype)
            flusher.clear()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            layer(x)
            e1.record()
            torch.cuda.synchronize()
            if it >= warmup:
                times.append(e0.elapsed_time(e1))
    return _trimmed_mean(times)


def benchmark_backward(layer, B, n, C, device, flusher, warmup, runs, dtype):
    layer.train()
    times = []
    for it in range(warmup + runs):
        x = torch.randn(B, n, C, device=device, dtype=torch.float32).to(dtype).requires_grad_(True)
        flusher.clear()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out = layer(x)
        out.sum().backward()
        e1.record()
        torch.cuda.synchronize()
        if it >= warmup:
            times.append(e0.elapsed_time(e1))
        for p in layer.parameters():
            p.grad = None
    return _trimmed_mean(times)


def _table(title, configs, make_fused, make_plain, bench, args, device, flusher, dtype):
    print(title)
    print("-" * 80)
    print(f"{'Batch':>6} {'Hidden':>6} {'n':>4} {'Fused (ms)':>12} {'Naive (ms)':>12} {'Speedup':>10}")
    print("-" * 80)
    for B, C, n in configs:
        fused = make_fused(C, n).to(device)
        plain = make_plain(C, n).to(device)
        tf = bench(fused, B, n, C, device, flusher, args.warmup, args.runs, dtype)
        tp = bench(plain, B, n, C, device, flusher, args.warmup, args.runs, torch.float32)
        print(f"{B:>6} {C:>6} {n:>4} {tf:>12.3f} {tp:>12.3f} {tp / tf:>9.2f}x", flush=True)
        del fused, plain
        torch.cuda.empty_cache()
    print()


def main():
    ap = argparse.ArgumentParser(description="Benchmark mHC Layer")
    ap.add_argument("--batch", type=int, default=64, help="Batch size")
    ap.add_argument("--hidden", type=int, default=1280, help="Hidden dimension")
    ap.add_argument("--expansion", type=int, default=4, help="Expansion rate (n)")
    ap.add_argument("--sinkhorn-iters", type=int, default=20, help="Sinkhorn iterations")
    ap.add_argument("--warmup", type=int, default=10, help="Warmup iterations")
    ap.add_argument("--runs", type=int, default=100, help="Benchmark runs")
    ap.add_argument("--backward", action="store_true", help="Benchmark backward pass too")
    ap.add_argument("--all-configs", action="store_true", help="Run all standard configs")
    ap.add_argument("--compute", choices=["bf16", "fp32", "bf16-io"], default="bf16",
                    help="fused layer: cast fp32 input to bf16 inside (default), exact fp32 kernels, or "
                         "bf16 activations in and out (the plain layer always runs fp32)")
    args = ap.parse_args()

    from mhc import MHCLayer

    device = torch.device("cuda")
    flusher = CacheFlusher(device)
    dtype = torch.bfloat16 if args.compute == "bf16-io" else torch.float32
    out_dtype = torch.bfloat16 if args.compute == "bf16-io" else None
    compute_dtype = torch.bfloat16 if args.compute == "bf16" else None
    if args.all_configs:
        configs = [(320, 1280, 4), (512, 1920, 4), (1280, 2560, 4), (2560, 1280, 4), (128, 1280, 8),
                   (256, 1280, 8), (32, 1280, 32), (64, 1280, 32), (128, 1280, 32)]
    else:
        configs = [(args.batch, args.hidden, args.expansion)]
    T = args.sinkhorn_iters

    print("mHC Layer Python Benchmark")
    print("=" * 80)
    print(f"Device: {torch.cuda.get_device_name(0)}")
    print(f"Sinkhorn iterations: {T}")
    print(f"Warmup: {args.warmup}, Runs: {args.runs}, fused-layer compute mode: {args.compute}")
    print()

    def fused(dynamic):
        return lambda C, n: MHCLayer(hidden_dim=C, expansion_rate=n, sinkhorn_iters=T, use_dynamic_h=dynamic,
                                     output_dtype=out_dtype, compute_dtype=compute_dtype)

    static_plain = lambda C, n: PlainStaticLayer(C, n, T)
    dynamic_plain = lambda C, n: PlainDynamicLayer(C, n, T)
    _table("Static H Path (shared H across batch)", configs, fused(False), static_plain,
           benchmark_forward, args, device, flusher, dtype)
    _table("Dynamic H Path (per-sample H)", configs, fused(True), dynamic_plain, benchmark_forward, args,
           device, flusher, dtype)
    if args.backward:
        _table("Backward Pass Static H (forward + backward)", configs, fused(False), static_plain,
               benchmark_backward, args, device, flusher, dtype)
        _table("Backward Pass Dynamic H Path (forward + backward)", configs, fused(True), dynamic_plain,
               benchmark_backward, args, device, flusher, dtype)


if __name__ == "__main__":
    main()
