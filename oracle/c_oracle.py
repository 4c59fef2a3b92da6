"""ctypes loader for the plain-C oracle (mhc_oracle.c).  Test infrastructure only.

All arrays are float64, C-contiguous numpy arrays.  ``logits``/``bias`` use the row order
[pre(n) | post(n) | res(n*n, row-major)], the same as the rows of phi_concat [D, nC].
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "libmhc_oracle.so"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libmhc_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(a):
    if a is None:
        return ctypes.c_void_p(None)
    assert a.dtype == np.float64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def _d(a):
    return None if a is None else np.ascontiguousarray(np.asarray(a, dtype=np.float64))


def dynamic_forward(x, w, phi, bias, alpha, T, eps, f_inject=None):
    x, w, phi, bias, alpha, f_inject = map(_d, (x, w, phi, bias, alpha, f_inject))
    B, n, C = x.shape
    y = np.empty_like(x)
    Hpre = np.empty((B, n)); Hpost = np.empty((B, n)); M = np.empty((B, n, n))
    rc = lib().mhc_oracle_dynamic_forward(_p(x), _p(w), _p(phi), _p(bias), _p(alpha), _p(f_inject),
                                          B, n, C, int(T), ctypes.c_double(eps), _p(y), _p(Hpre),
                                          _p(Hpost), _p(M))
    assert rc == 0
    return y, Hpre, Hpost, M


def dynamic_backward(x, dy, w, phi, bias, alpha, T, eps, f_inject=None):
    x, dy, w, phi, bias, alpha, f_inject = map(_d, (x, dy, w, phi, bias, alpha, f_inject))
    B, n, C = x.shape
    D = n * n + 2 * n
    dx = np.empty_like(x)
    df = np.empty((B, C)) if f_inject is not None else None
    dw = np.zeros(C)
    dphi = np.empty((D, n * C)); dbias = np.empty(D); dalpha = np.empty(3)
    rc = lib().mhc_oracle_dynamic_backward(_p(x), _p(dy), _p(w), _p(phi), _p(bias), _p(alpha),
                                           _p(f_inject), B, n, C, int(T), ctypes.c_double(eps),
                                           _p(dx), _p(df), _p(dw), _p(dphi), _p(dbias), _p(dalpha))
    assert rc == 0
    return dict(x=dx, f=df, w=dw, phi=dphi, bias=dbias, alpha=dalpha)


def static_forward(x, w, logits, T, eps, f_inject=None):
    x, w, logits, f_inject = map(_d, (x, w, logits, f_inject))
    B, n, C = x.shape
    y = np.empty_like(x)
    Hpre = np.empty(n); Hpost = np.empty(n); M = np.empty((n, n))
    rc = lib().mhc_oracle_static_forward(_p(x), _p(w), _p(logits), _p(f_inject), B, n, C, int(T),
                                         ctypes.c_double(eps), _p(y), _p(Hpre), _p(Hpost), _p(M))
    assert rc == 0
    return y, Hpre, Hpost, M


def static_backward(x, dy, w, logits, T, eps, f_inject=None):
    x, dy, w, logits, f_inject = map(_d, (x, dy, w, logits, f_inject))
    B, n, C = x.shape
    D = n * n + 2 * n
    dx = np.empty_like(x)
    df = np.empty((B, C)) if f_inject is not None else None
    dw = np.zeros(C)
    dlogits = np.empty(D)
    rc = lib().mhc_oracle_static_backward(_p(x), _p(dy), _p(w), _p(logits), _p(f_inject), B, n, C,
                                          int(T), ctypes.c_double(eps), _p(dx), _p(df), _p(dw),
                                          _p(dlogits))
    assert rc == 0
    return dict(x=dx, f=df, w=dw, logits=dlogits)


def sinkhorn_plain_forward(inp, T, eps):
    inp = _d(inp)
    rows, cols = inp.shape
    out = np.empty_like(inp)
    assert lib().mhc_oracle_sinkhorn_plain_forward(_p(inp), _p(out), rows, cols, int(T), ctypes.c_double(eps)) == 0
    return out


def sinkhorn_plain_backward(grad_out, inp, T, eps):
    grad_out, inp = _d(grad_out), _d(inp)
    rows, cols = inp.shape
    d_inp = np.empty_like(inp)
    assert lib().mhc_oracle_sinkhorn_plain_backward(_p(grad_out), _p(inp), _p(d_inp), rows, cols, int(T),
                                                    ctypes.c_double(eps)) == 0
    return d_inp


def rmsnorm_forward(inp, w, eps):
    inp, w = _d(inp), _d(w)
    rows, C = inp.shape
    out, rms = np.empty_like(inp), np.empty(rows)
    assert lib().mhc_oracle_rmsnorm_forward(_p(inp), _p(w), _p(out), _p(rms), rows, C, ctypes.c_double(eps)) == 0
    return out, rms


def rmsnorm_backward(grad, inp, w, rms):
    grad, inp, w, rms = _d(grad), _d(inp), _d(w), _d(rms)
    rows, C = inp.shape
    d_inp, d_w = np.empty_like(inp), np.empty(C)
    assert lib().mhc_oracle_rmsnorm_backward(_p(grad), _p(inp), _p(w), _p(rms), _p(d_inp), _p(d_w), rows, C) == 0
    return d_inp, d_w
