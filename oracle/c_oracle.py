"""ctypes loader for oracle/libgq_oracle.so (the plain-C restatement).

TEST INFRASTRUCTURE ONLY: used by tests/, the smoke check and the benchmark's
cpu_baseline leg.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    """Compile the C oracle in place (gcc + make) and return the library path."""
    subprocess.run(["make", "-C", _HERE, "-B", "libgq_oracle.so"], check=True, capture_output=True)
    return os.path.join(_HERE, "libgq_oracle.so")


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libgq_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.gqo_h2f.restype = ctypes.c_float
        _LIB.gqo_h2f.argtypes = [ctypes.c_uint16]
        _LIB.gqo_f2h.restype = ctypes.c_uint16
        _LIB.gqo_f2h.argtypes = [ctypes.c_float]
    return _LIB


def _p(a: np.ndarray):
    return ctypes.c_void_p(a.ctypes.data)


def num_threads() -> int:
    return int(lib().gqo_num_threads())


def quantize(w: np.ndarray, bits: int, group_size: int, round_mode: int = 0):
    assert w.dtype == np.float16 and w.ndim == 2 and w.flags.c_contiguous
    rows, k = w.shape
    ng = -(-k // group_size)
    nw = (group_size // (32 // bits)) * ng
    qw = np.empty((rows, nw), np.uint32)
    qs = np.empty((rows, ng), np.float16)
    rc = lib().gqo_quantize(_p(w), ctypes.c_int64(rows), ctypes.c_int64(k), bits, group_size,
                            round_mode, _p(qw), _p(qs))
    assert rc == 0, rc
    return qw, qs


def dequantize(qw: np.ndarray, qs: np.ndarray, k: int, bits: int, group_size: int):
    assert qw.dtype == np.uint32 and qs.dtype == np.float16
    qw = np.ascontiguousarray(qw)
    qs = np.ascontiguousarray(qs)
    rows = qw.shape[0]
    out = np.empty((rows, k), np.float16)
    rc = lib().gqo_dequantize(_p(qw), _p(qs), ctypes.c_int64(rows), ctypes.c_int64(k), bits,
                              group_size, _p(out))
    assert rc == 0, rc
    return out


def linear(x: np.ndarray, qw: np.ndarray, qs: np.ndarray, bits: int, group_size: int, bias=None,
           scratch=None, out=None):
    """float32 [M, N]; M <= 64."""
    assert x.dtype == np.float16 and x.ndim == 2 and x.flags.c_contiguous
    m, k = x.shape
    n = qw.shape[0]
    scratch = np.empty(m * k, np.float32) if scratch is None else scratch
    out = np.empty((m, n), np.float32) if out is None else out
    rc = lib().gqo_linear(_p(x), _p(qw), _p(qs), _p(bias) if bias is not None else None,
                          ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k), bits, group_size,
                          _p(scratch), _p(out))
    assert rc == 0, rc
    return out


def group_gemm(x: np.ndarray, qw: np.ndarray, qs: np.ndarray, indptr: np.ndarray, bits: int,
               group_size: int):
    assert x.dtype == np.float16 and x.flags.c_contiguous and indptr.dtype == np.int32
    rows, k = x.shape
    ne, n, _ = qw.shape
    scratch = np.empty(rows * k, np.float32)
    out = np.zeros((rows, n), np.float32)
    rc = lib().gqo_group_gemm(_p(x), _p(qw), _p(qs), _p(indptr), ctypes.c_int64(ne),
                              ctypes.c_int64(n), ctypes.c_int64(k), bits, group_size, _p(scratch),
                              _p(out))
    assert rc == 0, rc
    return out
