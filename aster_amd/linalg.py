"""`linalg.matmul`-shaped entry on top of the GEMM path: C[M,N] = A[M,K] @ B[K,N].

The reference's second consumer of its GEMM kernels is the linalg-to-AMDGCN route of
contrib/mlir-air, whose end-to-end test hands the kernel a row-major A[M,K] and a B that
was given as K x N and transposed on the host
(contrib/mlir-air/test/integration/test_linalg_matmul_e2e.py:52-60).  The kernels here
take B as N x K as well, so this helper does the same host-side step and then runs the
ordinary path through the C-ABI.
"""
from __future__ import annotations

import numpy as np

from . import gemm as _gemm
from .execution import GpuBuffer

_NP_OUT = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}


def matmul(a: np.ndarray, b_kxn: np.ndarray, out_dtype: str = "f32") -> np.ndarray:
    """A[M,K] (float16) times B[K,N] (float16) with fp32 accumulation on the GPU.

    Returns C[M,N] as float32 / float16, or raw bfloat16 bits (uint16) for "bf16".
    Raises ValueError on shape or dtype mismatch, like numpy's matmul does."""
    a = np.asarray(a)
    b_kxn = np.asarray(b_kxn)
    if a.ndim != 2 or b_kxn.ndim != 2:
        raise ValueError("matmul: both operands must be 2-D")
    if a.shape[1] != b_kxn.shape[0]:
        raise ValueError(f"matmul: shapes {a.shape} and {b_kxn.shape} do not chain")
    if a.dtype != np.float16 or b_kxn.dtype != np.float16:
        raise ValueError("matmul: operands must be float16")
    if out_dtype not in _NP_OUT:
        raise ValueError(f"matmul: unknown output dtype {out_dtype!r}")
    (M, K), N = a.shape, b_kxn.shape[1]
    if K % 8 != 0:
        raise ValueError("matmul: K must be a multiple of 8 (16-byte rows)")
    a = np.ascontiguousarray(a)
    b_nxk = np.ascontiguousarray(b_kxn.T)          # the host transpose of the reference's test
    c = np.zeros((M, N), dtype=_NP_OUT[out_dtype])
    if M == 0 or N == 0:
        return c
    plan = _gemm.GemmPlan.create(M, N, K, "f16", out_dtype)
    bufs = [GpuBuffer(x.nbytes) for x in (a, b_nxk, c)]
    try:
        bufs[0].copy_from_host(a)
        bufs[1].copy_from_host(b_nxk)
        plan.run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2].ptr_value)
        bufs[2].copy_to_host(c)
    finally:
        for buf in bufs:
            buf.free()
    return c
