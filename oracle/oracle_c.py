"""ctypes binding for the plain-C restatement (oracle_c.c).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_c.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _sz(v):
    return ctypes.c_size_t(int(v))


def corr1ord(W, X, Z):
    X = np.ascontiguousarray(X).ravel()
    lib().orc_corr1ord(_p(W), _sz(W.shape[0] // 4), _sz(W.shape[1]), _p(X), _sz(X.size), _p(Z))
    return Z


def corr1ord_bprop_W(dW, X, dZ):
    X = np.ascontiguousarray(X).ravel()
    lib().orc_corr1ord_bprop_W(_p(dW), _sz(dW.shape[0] // 4), _sz(dW.shape[1]), _p(X), _sz(X.size), _p(dZ))
    return dW


def corr1ord_bprop_X(dX, W, dZ):
    lib().orc_corr1ord_bprop_X(_p(dX), _sz(dX.shape[0]), _p(W), _sz(W.shape[0] // 4), _sz(W.shape[1]), _p(dZ))
    return dX


def poolrgn(U, R, ptype, want_argmax=False):
    P, F = R.shape[0], U.shape[1]
    pooled = np.empty((P, F * (2 if ptype == 3 else 1)), np.float32)
    amax = np.empty((P, F), np.uint32) if (want_argmax and ptype in (0, 3)) else None
    lib().orc_poolrgn(_p(U), _sz(F), _p(R), _sz(P), ctypes.c_int(R.shape[1] == 3), _p(pooled), _p(amax), ctypes.c_int(ptype))
    return pooled, amax


def poolrgn_bprop(dU, R, dP, amax, ptype):
    lib().orc_poolrgn_bprop(_p(dU), _sz(dU.shape[1]), _p(R), _sz(R.shape[0]), ctypes.c_int(R.shape[1] == 3),
                            _p(dP), _p(amax), ctypes.c_int(ptype))
    return dU


def scanpool(W, bias, X, R, ptype, want_argmax=False):
    X = np.ascontiguousarray(X).ravel()
    P, F = R.shape[0], W.shape[1]
    pooled = np.empty((P, F * (2 if ptype == 3 else 1)), np.float32)
    amax = np.empty((P, F), np.uint32) if (want_argmax and ptype in (0, 3)) else None
    bias = np.ascontiguousarray(bias, dtype=np.float32).ravel()
    lib().orc_scanpool(_p(W), _p(bias), _sz(W.shape[0] // 4), _sz(F), _p(X), _sz(X.size), _p(R), _sz(P),
                       ctypes.c_int(ptype), _p(pooled), _p(amax))
    return pooled, amax
