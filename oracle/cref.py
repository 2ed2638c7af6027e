"""ctypes binding of oracle/evo_ref.c (test infrastructure only).

Head-major fp64 numpy arrays in, fp64 arrays out.  See evo_ref.c for the formula and the
reference lines it follows (test.py:47-57; evoformer.py:285-288, 313-323, 450-462, 594-614).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force: bool = False) -> str:
    path = os.path.join(_HERE, "libevo_ref.so")
    if force or not os.path.exists(path):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libevo_ref.so"], stdout=subprocess.DEVNULL)
    return path


def _lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(build())
        dp = ctypes.POINTER(ctypes.c_double)
        _LIB.evo_ref_fwd.argtypes = [dp] * 5 + [ctypes.c_int] * 5 + [ctypes.c_double, dp, dp]
        _LIB.evo_ref_bwd.argtypes = [dp] * 6 + [ctypes.c_int] * 5 + [ctypes.c_double] + [dp] * 5
    return _LIB


def _p(a):
    if a is None:
        return ctypes.POINTER(ctypes.c_double)()
    assert a.dtype == np.float64 and a.flags.c_contiguous
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def fwd(q, k, v, bias=None, mask=None):
    """q,k,v [B,H,S,N,D]; bias [B,H,N,N]; mask [B,S,N] additive.  Returns (o, lse)."""
    B, H, S, N, D = q.shape
    o = np.empty_like(q)
    lse = np.empty((B, H, S, N))
    rc = _lib().evo_ref_fwd(_p(q), _p(k), _p(v), _p(bias), _p(mask), B, H, S, N, D,
                            float(D) ** -0.5, _p(o), _p(lse))
    assert rc == 0
    return o, lse


def bwd(q, k, v, do, bias=None, mask=None):
    """Returns dq, dk, dv, dbias (or None), dmask (or None)."""
    B, H, S, N, D = q.shape
    dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
    dbias = None if bias is None else np.empty((B, H, N, N))
    dmask = None if mask is None else np.empty((B, S, N))
    rc = _lib().evo_ref_bwd(_p(q), _p(k), _p(v), _p(bias), _p(mask), _p(do), B, H, S, N, D,
                            float(D) ** -0.5, _p(dq), _p(dk), _p(dv), _p(dbias), _p(dmask))
    assert rc == 0
    return dq, dk, dv, dbias, dmask
