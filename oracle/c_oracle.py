"""ctypes wrapper around oracle/libsa_oracle.so (TEST INFRASTRUCTURE ONLY)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def load():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "libsa_oracle.so")
        if not os.path.exists(path):
            subprocess.check_call(["make", "-C", _HERE, "-s"])
        _lib = ctypes.CDLL(path)
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def run(q, k, v, lens, context_size, back_contexts, sm_scale=None, d_out=None):
    """q/k/v/d_out: array-likes [B,H,T,D]; returns dict of float64 numpy arrays."""
    lib = load()
    qn, kn, vn = (np.ascontiguousarray(np.asarray(t, dtype=np.float64)) for t in (q, k, v))
    B, H, T, D = qn.shape
    s = float(D) ** -0.5 if sm_scale is None else float(sm_scale)
    ln = None if lens is None else np.ascontiguousarray(np.asarray(lens, dtype=np.int32))
    C = int(min(context_size, max(T, 1)))
    R = int(min(back_contexts, max(T, 1)))
    o = np.empty_like(qn)
    lse = np.empty((B, H, T))
    rc = lib.sa_oracle_forward(_ptr(qn), _ptr(kn), _ptr(vn), _ptr(ln) if ln is not None else None,
                               _ptr(o), _ptr(lse), B, H, T, D, C, R, ctypes.c_double(s))
    assert rc == 0
    out = {"O": o, "LSE": lse}
    if d_out is not None:
        g = np.ascontiguousarray(np.broadcast_to(np.asarray(d_out, dtype=np.float64), qn.shape))
        dq, dk, dv = np.empty_like(qn), np.empty_like(qn), np.empty_like(qn)
        rc = lib.sa_oracle_backward(_ptr(qn), _ptr(kn), _ptr(vn), _ptr(ln) if ln is not None else None,
                                    _ptr(o), _ptr(lse), _ptr(g), _ptr(dq), _ptr(dk), _ptr(dv),
                                    B, H, T, D, C, R, ctypes.c_double(s))
        assert rc == 0
        out.update(dQ=dq, dK=dk, dV=dv)
    return out
