"""ctypes front-end of the C oracle (oracle/lfw_oracle.c; the delta rule's oracle is oracle/dfw_ref.py).

TEST INFRASTRUCTURE ONLY.  Loads oracle/_build/liboracle.so, building it with gcc
when it is missing (the oracle is CPU code; building the checker is not using it).
"""
import ctypes
import os

import numpy as np

from . import build as _build

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_build.LIB):
            _build.build()
        _lib = ctypes.CDLL(_build.LIB)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f64(t):
    """torch tensor / ndarray -> contiguous float64 ndarray"""
    if hasattr(t, "detach"):
        t = t.detach().to("cpu").double().numpy()
    return np.ascontiguousarray(t, dtype=np.float64)


def lfw_forward(x, f, q, k, fk, s0):
    x, f, q, k, fk, s0 = map(_f64, (x, f, q, k, fk, s0))
    B, T, D = x.shape
    K = q.shape[-1]
    out = np.empty((B, T, D))
    nxt = np.empty((B, D, K))
    i64 = ctypes.c_int64
    rc = lib().lfw_oracle_forward(_p(x), _p(f), _p(q), _p(k), _p(fk), _p(s0),
                                  _p(out), _p(nxt), i64(B), i64(T), i64(D), i64(K))
    assert rc == 0
    return out, nxt


def lfw_backward(g_out, g_state, x, f, q, k, fk, s0):
    g_out, g_state, x, f, q, k, fk, s0 = map(_f64, (g_out, g_state, x, f, q, k, fk, s0))
    B, T, D = x.shape
    K = q.shape[-1]
    d_x, d_f = np.empty((B, T, D)), np.empty((B, T, D))
    d_q, d_k, d_fk = np.empty((B, T, K)), np.empty((B, T, K)), np.empty((B, T, K))
    d_s0 = np.empty((B, D, K))
    i64 = ctypes.c_int64
    rc = lib().lfw_oracle_backward(_p(g_out), _p(g_state), _p(x), _p(f), _p(q), _p(k),
                                   _p(fk), _p(s0), _p(d_x), _p(d_f), _p(d_q), _p(d_k),
                                   _p(d_fk), _p(d_s0), i64(B), i64(T), i64(D), i64(K))
    assert rc == 0
    return d_x, d_f, d_q, d_k, d_fk, d_s0
