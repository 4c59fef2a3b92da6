"""Writes golden input/output vectors from the reference's OWN naive PyTorch layers.

Run once, in the build container, where the reference tree is mounted read-only:

    python tests/golden/make_golden.py [/root/reference]

It imports (does not copy) two reference modules that need nothing but torch on the CPU -
src/python/benchmarks/bench_layer.py (NaiveMHCLayer, NaiveMHCLayerDynamic) and
src/python/tests/test_layer.py (_naive_mhc_dynamic) - runs them in fp64 on small seeded
inputs with every parameter randomised away from its init value, and stores inputs, outputs and
all autograd gradients as .npz next to this file.  The fixtures pin what only the reference's
text decides: row-then-column order of the Sinkhorn loop, eps added to the denominators, one
eps shared by both RMSNorms and Sinkhorn, the row-major reshape of the H_res projection, and
the [pre | post | res] ordering of the projection weights.  tests/test_oracle_golden.py checks
the oracle against them; the GPU parity tests reuse the same files.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _np(t):
    return t.detach().double().numpy()


def static_case(bench, tag, B, n, C, T, eps, seed):
    g = torch.Generator().manual_seed(seed)
    layer = bench.NaiveMHCLayer(C, n, sinkhorn_iters=T, eps=eps).double()
    with torch.no_grad():
        layer.rmsnorm_weight.copy_(1.0 + 0.5 * torch.randn(C, generator=g, dtype=torch.float64))
        layer.H_pre.copy_(torch.randn(n, generator=g, dtype=torch.float64))
        layer.H_post.copy_(torch.randn(n, generator=g, dtype=torch.float64))
        layer.H_res.copy_(torch.randn(n, n, generator=g, dtype=torch.float64))
    x = torch.randn(B, n, C, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(B, n, C, generator=g, dtype=torch.float64)
    y = layer(x)
    y.backward(dy)
    out = dict(B=B, n=n, C=C, T=T, eps=eps, x=_np(x), dy=_np(dy), y=_np(y), dx=_np(x.grad),
               w=_np(layer.rmsnorm_weight), H_pre=_np(layer.H_pre), H_post=_np(layer.H_post),
               H_res=_np(layer.H_res), dw=_np(layer.rmsnorm_weight.grad),
               dH_pre=_np(layer.H_pre.grad), dH_post=_np(layer.H_post.grad),
               dH_res=_np(layer.H_res.grad))
    np.savez(os.path.join(HERE, f"static_{tag}.npz"), **out)


def dynamic_case(bench, tag, B, n, C, T, eps, seed):
    """NaiveMHCLayerDynamic stores phi as [nC, n] / [nC, n*n]; the fixture keeps that layout."""
    g = torch.Generator().manual_seed(seed)
    layer = bench.NaiveMHCLayerDynamic(C, n, sinkhorn_iters=T, eps=eps).double()
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    with torch.no_grad():
        layer.rmsnorm_weight.copy_(1.0 + 0.5 * rnd(C))
        layer.phi_pre.copy_(0.3 * rnd(n * C, n))
        layer.phi_post.copy_(0.3 * rnd(n * C, n))
        layer.phi_res.copy_(0.3 * rnd(n * C, n * n))
        layer.b_pre.copy_(0.5 * rnd(n))
        layer.b_post.copy_(0.5 * rnd(n))
        layer.b_res.copy_(0.5 * rnd(n, n))
        layer.alpha_pre.fill_(0.7)
        layer.alpha_post.fill_(-0.4)
        layer.alpha_res.fill_(0.9)
    x = torch.randn(B, n, C, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(B, n, C, generator=g, dtype=torch.float64)
    y = layer(x)
    y.backward(dy)
    out = dict(B=B, n=n, C=C, T=T, eps=eps, x=_np(x), dy=_np(dy), y=_np(y), dx=_np(x.grad))
    for name, p in layer.named_parameters():
        out[name if name != "rmsnorm_weight" else "w"] = _np(p)
        out["d" + (name if name != "rmsnorm_weight" else "w")] = _np(p.grad)
    np.savez(os.path.join(HERE, f"dynamic_{tag}.npz"), **out)


def functional_case(tl, tag, B, n, C, T, eps, seed):
    """_naive_mhc_dynamic takes phi as [n, nC] / [n*n, nC] (MHCLayer's layout)."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    p = dict(w=1.0 + 0.5 * rnd(C), phi_pre=0.3 * rnd(n, n * C), phi_post=0.3 * rnd(n, n * C),
             phi_res=0.3 * rnd(n * n, n * C), alpha_pre=torch.tensor(0.6, dtype=torch.float64),
             alpha_post=torch.tensor(-0.5, dtype=torch.float64),
             alpha_res=torch.tensor(0.8, dtype=torch.float64), b_pre=0.5 * rnd(n),
             b_post=0.5 * rnd(n), b_res=0.5 * rnd(n, n))
    for v in p.values():
        v.requires_grad_(True)
    x = rnd(B, n, C).requires_grad_(True)
    dy = rnd(B, n, C)
    y = tl._naive_mhc_dynamic(x, p["w"], p["phi_pre"], p["phi_post"], p["phi_res"],
                              p["alpha_pre"], p["alpha_post"], p["alpha_res"], p["b_pre"],
                              p["b_post"], p["b_res"], T, eps)
    y.backward(dy)
    out = dict(B=B, n=n, C=C, T=T, eps=eps, x=_np(x), dy=_np(dy), y=_np(y), dx=_np(x.grad))
    for k, v in p.items():
        out[k] = _np(v)
        out["d" + k] = _np(v.grad)
    np.savez(os.path.join(HERE, f"functional_{tag}.npz"), **out)


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    bench = _load(os.path.join(ref, "src/python/benchmarks/bench_layer.py"), "ref_bench_layer")
    tl = _load(os.path.join(ref, "src/python/tests/test_layer.py"), "ref_test_layer")
    static_case(bench, "n4", B=3, n=4, C=16, T=20, eps=1e-5, seed=11)
    static_case(bench, "n8", B=2, n=8, C=24, T=5, eps=1e-3, seed=12)
    dynamic_case(bench, "n4", B=3, n=4, C=16, T=20, eps=1e-5, seed=21)
    dynamic_case(bench, "n8", B=2, n=8, C=32, T=7, eps=1e-3, seed=22)
    dynamic_case(bench, "n3", B=2, n=3, C=8, T=3, eps=1e-6, seed=23)
    functional_case(tl, "n4", B=2, n=4, C=16, T=3, eps=1e-5, seed=31)
    functional_case(tl, "n16", B=2, n=16, C=4, T=20, eps=1e-6, seed=32)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
