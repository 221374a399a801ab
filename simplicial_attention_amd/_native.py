"""ctypes binding of libsa2.so, the C-ABI library declared in include/sa2.h.

The library is built in-tree by ``simplicial_attention_amd/csrc/Makefile`` (hipcc,
gfx950).  There is no fallback: if the shared object is missing or a call fails,
an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import threading

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'csrc')
LIB_PATH = os.path.join(_CSRC, 'libsa2.so')
PROF_LIB_PATH = os.path.join(_CSRC, 'libsa2_prof.so')   # -DSA2_PROFILING build, for bench.py only

SA2_OK = 0
SA2_BF16 = 0
STATUS_NAMES = {
    1: 'SA2_ERR_NULL_POINTER',
    2: 'SA2_ERR_BAD_SHAPE',
    3: 'SA2_ERR_UNSUPPORTED',
    4: 'SA2_ERR_ALIGNMENT',
    5: 'SA2_ERR_LAUNCH',
}

EXPORTS = ('sa2_version', 'sa2_last_error', 'sa2_supported', 'sa2_saved_t_bytes', 'sa2_saved_m_bytes', 'sa2_fwd',
           'sa2_bwd_delta', 'sa2_bwd_workspace_bytes', 'sa2_bwd_workspace_bytes_with_saved', 'sa2_bwd_dq_dkv2', 'sa2_bwd_dkv1', 'sa2_bwd',
           'sa2_bwd_noalloc_scratch_bytes', 'sa2_bwd_noalloc',
           'sa2_qkv_norm_fwd', 'sa2_qkv_norm_bwd_workspace_bytes', 'sa2_qkv_norm_bwd')


class Sa2Error(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f'{STATUS_NAMES.get(status, status)}: {message}')
        self.status = status


class Problem(ctypes.Structure):
    _fields_ = [('batch', ctypes.c_int32), ('seq_len', ctypes.c_int32), ('heads', ctypes.c_int32),
                ('kv_heads', ctypes.c_int32), ('dim_head', ctypes.c_int32), ('w1', ctypes.c_int32),
                ('w2', ctypes.c_int32), ('causal', ctypes.c_int32), ('scale', ctypes.c_float),
                ('dtype', ctypes.c_int32)]


class TensorArg(ctypes.Structure):
    _fields_ = [('ptr', ctypes.c_void_p), ('stride_b', ctypes.c_int64), ('stride_n', ctypes.c_int64),
                ('stride_h', ctypes.c_int64)]


class Saved(ctypes.Structure):
    """sa2_saved: optional forward by-products (per-offset T and its reference)."""
    _fields_ = [('t', ctypes.c_void_p), ('m', ctypes.c_void_p)]


_lib = None
_prof_lib = None
_lock = threading.Lock()


def build(verbose: bool = False) -> str:
    """Compile libsa2.so for gfx950 (always recompiles)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(['make', '-B', '-C', _CSRC, 'libsa2.so', 'libsa2_prof.so'], stdout=out, stderr=out)
    return LIB_PATH


def _declare(lib: ctypes.CDLL) -> ctypes.CDLL:
    P, T, F, V = ctypes.POINTER(Problem), ctypes.POINTER(TensorArg), ctypes.c_void_p, ctypes.c_void_p
    S = ctypes.POINTER(Saved)
    I64 = ctypes.c_int64
    for name in ('sa2_saved_t_bytes', 'sa2_saved_m_bytes', 'sa2_bwd_workspace_bytes', 'sa2_bwd_workspace_bytes_with_saved', 'sa2_qkv_norm_bwd_workspace_bytes',
                 'sa2_bwd_noalloc_scratch_bytes'):
        getattr(lib, name).restype = I64
        getattr(lib, name).argtypes = [P]
    lib.sa2_version.restype = ctypes.c_int
    lib.sa2_version.argtypes = []
    lib.sa2_last_error.restype = ctypes.c_char_p
    lib.sa2_last_error.argtypes = []
    lib.sa2_supported.restype = ctypes.c_int
    lib.sa2_supported.argtypes = [ctypes.c_int32] * 4
    lib.sa2_fwd.restype = ctypes.c_int
    lib.sa2_fwd.argtypes = [P, T, T, T, T, T, T, T, F, S, V]
    lib.sa2_bwd_delta.restype = ctypes.c_int
    lib.sa2_bwd_delta.argtypes = [P, T, T, T, F, V]
    lib.sa2_bwd_dq_dkv2.restype = ctypes.c_int
    lib.sa2_bwd_dq_dkv2.argtypes = [P, T, T, T, T, T, T, F, F, S, T, T, T, V, I64, V]
    lib.sa2_bwd_dkv1.restype = ctypes.c_int
    lib.sa2_bwd_dkv1.argtypes = [P, T, T, T, T, T, T, F, F, T, T, V]
    lib.sa2_bwd.restype = ctypes.c_int
    lib.sa2_bwd.argtypes = [P, T, T, T, T, T, T, T, T, F, S, F, T, T, T, T, T, V, I64, V]
    lib.sa2_bwd_noalloc.restype = ctypes.c_int
    lib.sa2_bwd_noalloc.argtypes = [P, T, T, T, T, T, T, T, T, F, S, T, T, T, T, T, V]
    lib.sa2_qkv_norm_fwd.restype = ctypes.c_int
    lib.sa2_qkv_norm_fwd.argtypes = [P, V, I64, V, V, V, V, V, ctypes.c_float, T, T, T, T, T, F, V]
    lib.sa2_qkv_norm_bwd.restype = ctypes.c_int
    lib.sa2_qkv_norm_bwd.argtypes = [P, V, I64, V, V, V, V, V, T, T, T, T, T, F, V, F, V, I64, V]
    return lib


def _missing(path: str) -> FileNotFoundError:
    return FileNotFoundError(f'{path} is missing: build it with `make -C {_CSRC}` '
                             '(or `python -c "import __graft_entry__ as g; g.build()"`)')


def load() -> ctypes.CDLL:
    """Load libsa2.so and declare its prototypes.  Raises if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise _missing(LIB_PATH)
            _lib = _declare(ctypes.CDLL(LIB_PATH))
        return _lib


def load_profiling() -> ctypes.CDLL:
    """The -DSA2_PROFILING build of the same sources: it honours SA2_BWD_PASS=first (launch only the
    MFMA kernel of the dQ/dK2/dV2 entry point, results incomplete).  For kernel timing only."""
    global _prof_lib
    with _lock:
        if _prof_lib is None:
            if not os.path.exists(PROF_LIB_PATH):
                raise _missing(PROF_LIB_PATH)
            _prof_lib = _declare(ctypes.CDLL(PROF_LIB_PATH))
        return _prof_lib


def check(status: int) -> None:
    if status != SA2_OK:
        raise Sa2Error(status, load().sa2_last_error().decode())


def tensor_arg(t) -> TensorArg:
    """(b, n, h, d) torch tensor with unit innermost stride -> sa2_tensor."""
    assert t.dim() == 4 and t.stride(3) == 1
    return TensorArg(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def problem(batch, seq_len, heads, kv_heads, dim_head, w1, w2, causal, scale) -> Problem:
    return Problem(batch, seq_len, heads, kv_heads, dim_head, int(w1), int(w2), int(bool(causal)), float(scale), SA2_BF16)


def saved_arg(t, m) -> Saved:
    """Device tensors for the forward's per-offset T (bf16) and reference (fp32) -> sa2_saved."""
    return Saved(t.data_ptr(), m.data_ptr())
