"""ctypes front end of the C oracle (oracle/ttt_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Used by tests (second checker, pinned against the numpy oracle) and by bench.py's
`cpu_baseline` leg (the timed host-CPU port of the reference path).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "_build", "libttt_oracle.so")


def build(force: bool = False) -> str:
    if force or not os.path.exists(LIB):
        subprocess.run(["make", "-C", HERE] + (["-B"] if force else []), check=True,
                       capture_output=True)
    return LIB


_lib = None


def _load():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def linear_fwd(W0, b0, xq, xk, xv, token_eta, lr, gamma, beta, K=16, eps=1e-6, dtype=np.float32,
               nthreads=1):
    """Returns (out, W_out [B,H,d,d], b_out [B,H,d]) computed in `dtype` (float32 or float64)."""
    suf = {np.float32: "f32", np.float64: "f64"}[dtype]
    a = [np.ascontiguousarray(x, dtype=dtype) for x in (xq, xk, xv, W0, b0, token_eta, lr, gamma, beta)]
    B, H, seq, d = a[0].shape
    out = np.empty_like(a[0])
    W = np.empty((B, H, d, d), dtype)
    b = np.empty((B, H, d), dtype)
    fn = getattr(_load(), "ttt_oracle_linear_fwd_" + suf)
    real = C.c_float if dtype == np.float32 else C.c_double
    fn.argtypes = [C.c_int] * 5 + [C.c_void_p] * 9 + [real] + [C.c_void_p] * 3 + [C.c_int]
    fn.restype = None
    fn(B, H, seq, d, K, *[_p(x) for x in a], real(eps), _p(out), _p(W), _p(b), nthreads)
    return out, W, b


def linear_bwd(W0, b0, xq, xk, xv, token_eta, lr, gamma, beta, d_out, K=16, eps=1e-6, dtype=np.float32,
               nthreads=1, d_W_out=None, d_b_out=None):
    """All nine gradients of the TTT-Linear inner loop, computed in `dtype`; d_W_out [B,H,d,d], d_b_out [B,H,d]:
    upstream gradients of the final state (None = zero).
    Returns a dict with the keys of ttt_oracle.linear_backward."""
    suf = {np.float32: "f32", np.float64: "f64"}[dtype]
    a = [np.ascontiguousarray(x, dtype=dtype) for x in (xq, xk, xv, W0, b0, token_eta, lr, gamma, beta)]
    go = np.ascontiguousarray(d_out, dtype=dtype)
    B, H, seq, d = a[0].shape
    assert seq % K == 0 and a[3].ndim == 3
    g = dict(d_xq=np.empty_like(a[0]), d_xk=np.empty_like(a[0]), d_xv=np.empty_like(a[0]),
             d_W0=np.empty((B, H, d, d), dtype), d_b0=np.empty((B, H, d), dtype), d_lr=np.empty((B, H, seq), dtype),
             d_token_eta=np.empty(seq, dtype), d_gamma=np.empty((H, d), dtype), d_beta=np.empty((H, d), dtype))
    fn = getattr(_load(), "ttt_oracle_linear_bwd_" + suf)
    real = C.c_float if dtype == np.float32 else C.c_double
    fn.argtypes = [C.c_int] * 5 + [C.c_void_p] * 9 + [real] + [C.c_void_p] * 12 + [C.c_int]
    fn.restype = None
    up = [None if x is None else np.ascontiguousarray(x, dtype=dtype) for x in (d_W_out, d_b_out)]
    fn(B, H, seq, d, K, *[_p(x) for x in a], real(eps), _p(go), *[None if x is None else _p(x) for x in up],
       *[_p(g[k]) for k in (
        "d_xq", "d_xk", "d_xv", "d_W0", "d_b0", "d_lr", "d_token_eta", "d_gamma", "d_beta")], nthreads)
    return g


def mlp_fwd(W1, b1, W2, b2, xq, xk, xv, token_eta, lr, gamma, beta, K=16, eps=1e-6, dtype=np.float32,
            nthreads=1):
    suf = {np.float32: "f32", np.float64: "f64"}[dtype]
    a = [np.ascontiguousarray(x, dtype=dtype)
         for x in (xq, xk, xv, W1, b1, W2, b2, token_eta, lr, gamma, beta)]
    B, H, seq, d = a[0].shape
    m = a[3].shape[-1]
    out = np.empty_like(a[0])
    o = [np.empty((B, H, d, m), dtype), np.empty((B, H, m), dtype),
         np.empty((B, H, m, d), dtype), np.empty((B, H, d), dtype)]
    fn = getattr(_load(), "ttt_oracle_mlp_fwd_" + suf)
    real = C.c_float if dtype == np.float32 else C.c_double
    fn.argtypes = [C.c_int] * 6 + [C.c_void_p] * 11 + [real] + [C.c_void_p] * 5 + [C.c_int]
    fn.restype = None
    fn(B, H, seq, d, m, K, *[_p(x) for x in a], real(eps), _p(out), *[_p(x) for x in o], nthreads)
    return (out, *o)
