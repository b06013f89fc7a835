"""ctypes binding of the C restatement ``egs_oracle.c`` (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libegs_oracle.so")
_lib = None

W_EIJ, W_EJI = 0, 1


def build() -> str:
    subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "libegs_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        dp = ctypes.POINTER(ctypes.c_double)
        ip = ctypes.POINTER(ctypes.c_int64)
        ints = [ctypes.c_int] * 7
        for name in ("egs_oracle_gather", "egs_oracle_scatter", "egs_oracle_dw"):
            fn = getattr(_lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [fp, fp, ip, dp] + ints
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _i(a):
    a = np.ascontiguousarray(a, dtype=np.int64)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))


def _d(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def gather(X, W, Ind, w_layout=W_EIJ):
    B, T, I = X.shape
    _, E, K = Ind.shape
    J = W.shape[2] if w_layout == W_EIJ else W.shape[1]
    X, xp = _f(X); W, wp = _f(W); Ind, ip = _i(Ind)
    Y = np.empty((B, E, K, J), dtype=np.float64)
    rc = lib().egs_oracle_gather(xp, wp, ip, _d(Y), B, T, E, K, I, J, w_layout)
    if rc:
        raise IndexError("Ind out of range")
    return Y


def scatter(Y, W, Ind, T, w_layout=W_EJI):
    B, E, K, J = Y.shape
    I = W.shape[2] if w_layout == W_EJI else W.shape[1]
    Y, yp = _f(Y); W, wp = _f(W); Ind, ip = _i(Ind)
    out = np.empty((B, T, I), dtype=np.float64)
    rc = lib().egs_oracle_scatter(yp, wp, ip, _d(out), B, T, E, K, I, J, w_layout)
    if rc:
        raise IndexError("Ind out of range")
    return out


def dw(Xs, Ys, Ind, dw_layout=W_EIJ):
    B, T, I = Xs.shape
    _, E, K, J = Ys.shape
    Xs, xp = _f(Xs); Ys, yp = _f(Ys); Ind, ip = _i(Ind)
    shape = (E, I, J) if dw_layout == W_EIJ else (E, J, I)
    dW = np.empty(shape, dtype=np.float64)
    rc = lib().egs_oracle_dw(xp, yp, ip, _d(dW), B, T, E, K, I, J, dw_layout)
    if rc:
        raise IndexError("Ind out of range")
    return dW
