"""ctypes access to oracle/sb_oracle.c (float64 brute force).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libsb_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        dp = C.POINTER(C.c_double)
        _lib.sb_oracle_forward.argtypes = [dp, dp, dp, C.c_int, C.c_int, C.c_double, C.c_int, dp, dp, dp]
        _lib.sb_oracle_backward.argtypes = [dp, dp, dp, dp, dp, C.c_int, C.c_int, C.c_double, C.c_int,
                                            dp, dp, dp]
    return _lib


def _p(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


def forward(q, k, v, scale, attend_current=False):
    """q,k,v: [T, D] array-likes -> (o [T,D], rem [T], A [T,T]) float64."""
    q, k, v = (np.ascontiguousarray(x, dtype=np.float64) for x in (q, k, v))
    T, D = q.shape
    o, rem, A = np.empty((T, D)), np.empty(T), np.empty((T, T))
    _load().sb_oracle_forward(_p(q), _p(k), _p(v), T, D, float(scale), int(attend_current), _p(o), _p(rem), _p(A))
    return o, rem, A


def backward(q, k, v, do, drem, scale, attend_current=False):
    q, k, v, do, drem = (np.ascontiguousarray(x, dtype=np.float64) for x in (q, k, v, do, drem))
    T, D = q.shape
    dq, dk, dv = np.empty((T, D)), np.empty((T, D)), np.empty((T, D))
    _load().sb_oracle_backward(_p(q), _p(k), _p(v), _p(do), _p(drem), T, D, float(scale),
                               int(attend_current), _p(dq), _p(dk), _p(dv))
    return dq, dk, dv
