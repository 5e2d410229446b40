"""ctypes loader for oracle/libmhffn_scalar.so (scalar C loops, double).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmhffn_scalar.so")


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libmhffn_scalar.so"])
    return _SO


def _lib():
    lib = ctypes.CDLL(build())
    dp = ctypes.POINTER(ctypes.c_double)
    lib.mhffn_scalar_forward.argtypes = [dp] * 6 + [ctypes.c_int] * 7
    lib.mhffn_scalar_backward.argtypes = [dp] * 11 + [ctypes.c_int] * 7
    return lib


def _p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def forward(Q, K, U, V, R):
    """numpy float64 in, float64 out."""
    Q, K, U, V, R = (np.ascontiguousarray(a, dtype=np.float64) for a in (Q, K, U, V, R))
    B, H, S, dh = Q.shape
    Hk, E, de, _ = K.shape
    O = np.empty_like(Q)
    _lib().mhffn_scalar_forward(_p(Q), _p(K), _p(U), _p(V), _p(R), _p(O), B, H, Hk, S, dh, E, de)
    return O


def backward(Q, K, U, V, R, dO):
    Q, K, U, V, R, dO = (np.ascontiguousarray(a, dtype=np.float64) for a in (Q, K, U, V, R, dO))
    B, H, S, dh = Q.shape
    Hk, E, de, _ = K.shape
    dQ, dK, dU, dV, dR = (np.empty_like(a) for a in (Q, K, U, V, R))
    _lib().mhffn_scalar_backward(_p(Q), _p(K), _p(U), _p(V), _p(R), _p(dO),
                                 _p(dQ), _p(dK), _p(dU), _p(dV), _p(dR), B, H, Hk, S, dh, E, de)
    return dQ, dK, dU, dV, dR
