"""ctypes front end of oracle/sa2_oracle.c (fp64 loops).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'libsa2_oracle.so')
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/sa2_oracle.c with gcc (through oracle/Makefile)."""
    if force or not os.path.exists(_LIB_PATH):
        if force and os.path.exists(_LIB_PATH):
            os.remove(_LIB_PATH)
        subprocess.check_call(['make', '-s', '-C', _HERE, 'libsa2_oracle.so'])
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        dp = ctypes.POINTER(ctypes.c_double)
        _lib.sa2_oracle_fwd.argtypes = [dp] * 7 + [ctypes.c_int] * 6 + [ctypes.c_double]
        _lib.sa2_oracle_fwd.restype = ctypes.c_int
        _lib.sa2_oracle_bwd.argtypes = [dp] * 13 + [ctypes.c_int] * 6 + [ctypes.c_double]
        _lib.sa2_oracle_bwd.restype = ctypes.c_int
    return _lib


def _np(t):
    return np.ascontiguousarray(t.detach().cpu().double().numpy())


def _ptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def fwd_bwd(q, k1, k2, v1, v2, dout, w1, w2, scale=None):
    """All tensors (b, n, h, d).  Returns fp64 torch tensors
    ``out, lse[b,h,n], (dq, dk1, dk2, dv1, dv2)``."""
    lib = _load()
    b, n, h, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    arrs = [_np(t) for t in (q, k1, k2, v1, v2)]
    out = np.zeros((b, n, h, d))
    lse = np.zeros((b, h, n))
    lib.sa2_oracle_fwd(*[_ptr(a) for a in arrs], _ptr(out), _ptr(lse), b, n, h, d, w1, w2, scale)
    grads = None
    if dout is not None:
        do = _np(dout)
        g = [np.zeros((b, n, h, d)) for _ in range(5)]
        lib.sa2_oracle_bwd(*[_ptr(a) for a in arrs], _ptr(out), _ptr(do), _ptr(lse),
                           *[_ptr(a) for a in g], b, n, h, d, w1, w2, scale)
        grads = tuple(torch.from_numpy(a) for a in g)
    return torch.from_numpy(out), torch.from_numpy(lse), grads
