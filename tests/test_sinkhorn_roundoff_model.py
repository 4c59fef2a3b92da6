"""Float32 model (NumPy, no GPU) of the n > 8 Sinkhorn forward in scaling form and its exact
backward, as csrc/sinkhorn_device.h (SkWg) runs them: M = diag(u) E diag(v), the denominators
rho_t = u (E v) + eps and s_t = v (E^T u) + eps kept per iteration, the reverse sweep dividing by
them and unwinding u, v with them.

It documents where a round-off that grew with the iteration count came from.  With the
denominators formed by a fused multiply-add (one rounding) the converged iteration does not settle:
on some rows and columns the denominators stay one ulp off 1 for ever, u and v keep drifting
against each other, and the reverse sweep - which divides by those denominators in every
iteration - moves away from the float64 result by about 2e-8 per iteration.  With product and sum
rounded separately the denominators reach exactly 1 and the error is flat.  The kernel uses the
unfused form in its fp32 tier; tests/test_gpu_parity.py checks the flat error on the GPU."""
import numpy as np

f32, f64 = np.float32, np.float64


def forward(E, T, eps, dt, fused):
    E = E.astype(dt)
    n = E.shape[0]
    u, v = np.ones(n, dt), np.ones(n, dt)
    rho, s = [], []

    def mul_add(a, b):
        if dt is f64 or not fused:
            return ((a * b).astype(dt) + dt(eps)).astype(dt)
        return (a.astype(f64) * b.astype(f64) + eps).astype(f32)  # exact product, one rounding

    for _ in range(T):
        rr = mul_add(u, (E * v[None, :]).sum(1, dtype=dt))
        u = (u / rr).astype(dt)
        sc = mul_add(v, (E * u[:, None]).sum(0, dtype=dt))
        v = (v / sc).astype(dt)
        rho.append(rr)
        s.append(sc)
    return u, v, rho, s


def backward(E, d, u, v, rho, s, dt):
    E, d = E.astype(dt), d.astype(dt).copy()
    for t in range(len(rho) - 1, -1, -1):
        cd = (d * u[:, None] * E).sum(0, dtype=dt)
        d = (d - cd[None, :] * v[None, :]).astype(dt)
        rdot = u * (d * E * v[None, :]).sum(1, dtype=dt)
        d = ((d / s[t][None, :] - rdot[:, None]) / rho[t][:, None]).astype(dt)
        v, u = (v * s[t]).astype(dt), (u * rho[t]).astype(dt)
    return d * E


def _errors(n, fused, seed=0):
    rng = np.random.default_rng(seed)
    E = np.exp(0.7 * rng.standard_normal((n, n)))
    dM = rng.standard_normal((n, n))
    out = []
    for T in (20, 256):
        ref = backward(E, dM, *forward(E, T, 1e-6, f64, False), f64)
        got = backward(E, dM, *forward(E, T, 1e-6, f32, fused), f32)
        out.append(np.abs(got - ref).max() / np.abs(ref).max())
    return out


def test_unfused_denominators_settle_and_the_backward_error_is_flat():
    for n in (16, 32):
        _, _, rho, s = forward(np.exp(0.7 * np.random.default_rng(0).standard_normal((n, n))), 256, 1e-6, f32, False)
        assert all((r == 1).all() for r in rho[200:]) and all((c == 1).all() for c in s[200:])
        e20, e256 = _errors(n, fused=False)
        assert e20 < 1e-6 and e256 < 1e-6 and e256 < 2 * e20


def test_fused_denominators_keep_drifting_and_the_backward_error_grows():
    grew = 0
    for n in (16, 32):
        for seed in range(4):
            rng = np.random.default_rng(seed)
            _, _, rho, s = forward(np.exp(0.7 * rng.standard_normal((n, n))), 256, 1e-6, f32, True)
            stuck = any((r != 1).any() for r in rho[200:]) or any((c != 1).any() for c in s[200:])
            e20, e256 = _errors(n, fused=True, seed=seed)
            grew += stuck and e256 > 4 * e20
    assert grew >= 4  # most inputs: the drift is the rule, not a corner case
