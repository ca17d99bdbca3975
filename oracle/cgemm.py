"""ctypes wrapper of the C restatement (cgemm.c).  Test infrastructure."""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "_build", "liboracle_gemm.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile cgemm.c with the Makefile next to it (gcc, OpenMP)."""
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _DIR] + (["-B"] if force else []), check=True,
                       capture_output=True)
    return _SO


def load():
    global _lib
    if _lib is None:
        build()
        lib = C.CDLL(_SO)
        lib.oracle_gemm_f32.restype = C.c_int
        lib.oracle_gemm_f32.argtypes = [C.c_void_p] * 3 + [C.c_int64] * 3
        lib.oracle_gemm_raw.restype = C.c_int
        lib.oracle_gemm_raw.argtypes = ([C.c_void_p] * 3 + [C.c_int64] * 3 + [C.c_int]
                                        + [C.c_int64] * 2 + [C.c_void_p] * 2)
        _lib = lib
    return _lib


def gemm_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    M, K = a.shape
    N = b.shape[0]
    c = np.empty((M, N), dtype=np.float32)
    rc = load().oracle_gemm_f32(a.ctypes.data, b.ctypes.data, c.ctypes.data, M, N, K)
    assert rc == 0
    return c


def gemm_raw(a_raw: np.ndarray, b_raw: np.ndarray, dtype: int, M: int, N: int, K: int,
             mx_a=None, mx_b=None) -> np.ndarray:
    """Decode + multiply on raw storage bytes; returns fp32 [M, N]."""
    a_raw = np.ascontiguousarray(a_raw)
    b_raw = np.ascontiguousarray(b_raw)
    c = np.empty((M, N), dtype=np.float32)
    lda = a_raw.nbytes // max(M, 1)
    ldb = b_raw.nbytes // max(N, 1)
    pa = np.ascontiguousarray(mx_a).ctypes.data if mx_a is not None else None
    pb = np.ascontiguousarray(mx_b).ctypes.data if mx_b is not None else None
    rc = load().oracle_gemm_raw(a_raw.ctypes.data, b_raw.ctypes.data, c.ctypes.data, M, N, K,
                                dtype, lda, ldb, pa, pb)
    assert rc == 0
    return c
