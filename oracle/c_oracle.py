"""ctypes binding of oracle/dwn_oracle.c (test infrastructure, see oracle/__init__.py)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libdwn_oracle.so")
_lib = None


def build():
    """Compile the C restatement (gcc, a second or two)."""
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        f32p = ctypes.POINTER(ctypes.c_float)
        i32p = ctypes.POINTER(ctypes.c_int32)
        _lib.oracle_dwn_layer_forward.argtypes = [f32p, i32p, f32p, f32p] + [ctypes.c_int] * 5
        _lib.oracle_dwn_layer_forward.restype = None
        _lib.oracle_dwn_layer_backward.argtypes = (
            [f32p, i32p, f32p, f32p, ctypes.c_double, ctypes.c_double, f32p, f32p] + [ctypes.c_int] * 5)
        _lib.oracle_dwn_layer_backward.restype = None
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def dwn_layer_forward(x, idx, luts):
    """x [B,I], idx [N,k], luts [N,O,L] -> y [B,N,O] float32."""
    x, xp = _f(x); luts, lp = _f(luts)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    B, I = x.shape; N, k = idx.shape; O = luts.shape[1]
    y = np.empty((B, N, O), dtype=np.float32)
    lib().oracle_dwn_layer_forward(xp, idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), lp,
                                   y.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), B, I, N, k, O)
    return y


def dwn_layer_backward(x, idx, luts, gy, alpha, beta):
    """-> gx [B,I], gl [N,O,L] float32 (double accumulation inside, like the reference's CPU path)."""
    x, xp = _f(x); luts, lp = _f(luts); gy, gp = _f(gy)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    B, I = x.shape; N, k = idx.shape; O = luts.shape[1]
    gx = np.empty((B, I), dtype=np.float32)
    gl = np.empty(luts.shape, dtype=np.float32)
    lib().oracle_dwn_layer_backward(xp, idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), lp, gp,
                                    float(alpha), float(beta),
                                    gx.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                    gl.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), B, I, N, k, O)
    return gx, gl
