"""ctypes front end of the C loop restatement (sepcorr_loops.c).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libsepcorr_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "all"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _sfx(dtype):
    return {np.dtype(np.float32): "_f32", np.dtype(np.float64): "_f64"}[np.dtype(dtype)]


def max_argmax_avg_forward(f1, f2):
    f1 = np.ascontiguousarray(f1); f2 = np.ascontiguousarray(f2)
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    out_u = np.empty((B, H1, W1, 2, H2), f1.dtype)
    out_v = np.empty((B, H1, W1, 2, W2), f1.dtype)
    am_u = np.empty((B, H1, W1, 1, H2), np.int32)
    am_v = np.empty((B, H1, W1, 1, W2), np.int32)
    getattr(lib(), "sep_max_argmax_avg_forward" + _sfx(f1.dtype))(
        _p(f1), _p(f2), _p(out_u), _p(out_v), _p(am_u), _p(am_v), B, H1, W1, H2, W2, C)
    return out_u, out_v, am_u, am_v


def compression_forward(f1, f2, a_u, a_v):
    f1, f2, a_u, a_v = (np.ascontiguousarray(x) for x in (f1, f2, a_u, a_v))
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    K = a_u.shape[3]
    cu = np.empty((B, H1, W1, K, H2), f1.dtype)
    cv = np.empty((B, H1, W1, K, W2), f1.dtype)
    getattr(lib(), "sep_compression_forward" + _sfx(f1.dtype))(
        _p(f1), _p(f2), _p(a_u), _p(a_v), _p(cu), _p(cv), B, H1, W1, H2, W2, C, K)
    return cu, cv


def max_argmax_avg_backward(f1, f2, am_u, am_v, g_u, g_v):
    f1, f2, g_u, g_v = (np.ascontiguousarray(x) for x in (f1, f2, g_u, g_v))
    am_u = np.ascontiguousarray(am_u, np.int32); am_v = np.ascontiguousarray(am_v, np.int32)
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    d1 = np.empty_like(f1); d2 = np.empty_like(f2)
    getattr(lib(), "sep_max_argmax_avg_backward" + _sfx(f1.dtype))(
        _p(f1), _p(f2), _p(am_u), _p(am_v), _p(g_u), _p(g_v), _p(d1), _p(d2), B, H1, W1, H2, W2, C)
    return d1, d2


def compression_backward(f1, f2, a_u, a_v, g_cu, g_cv):
    f1, f2, a_u, a_v, g_cu, g_cv = (np.ascontiguousarray(x) for x in (f1, f2, a_u, a_v, g_cu, g_cv))
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    K = a_u.shape[3]
    d1 = np.empty_like(f1); d2 = np.empty_like(f2)
    da_u = np.empty_like(a_u); da_v = np.empty_like(a_v)
    getattr(lib(), "sep_compression_backward" + _sfx(f1.dtype))(
        _p(f1), _p(f2), _p(a_u), _p(a_v), _p(g_cu), _p(g_cv), _p(d1), _p(d2), _p(da_u), _p(da_v),
        B, H1, W1, H2, W2, C, K)
    return d1, d2, da_u, da_v
