"""GEMM oracle: C[M,N] = epilogue(A[M,K] . B[N,K]^T).  Test infrastructure.

The value is the reference's own check,
`A.astype(np.float32) @ B.astype(np.float32).T`
(contrib/kittens/test/bench/bench_harness.py:821, 1837), applied to the
dequantised operands.  The epilogue (per-tensor scales, bias, output cast) has
no counterpart in the reference; it is defined here as
`cast(acc * (scale_a * scale_b) + bias)` with fp32 arithmetic and RNE casts.
"""

from __future__ import annotations

from typing import Optional

import numpy as np

from . import formats as F

F16, BF16, FP8_E4M3, MXFP4, F32 = 0, 1, 2, 3, 4


def gemm_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """The reference formula verbatim: fp32 operands, fp32 BLAS."""
    return a.astype(np.float32) @ b.astype(np.float32).T


def gemm_f64(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Same product accumulated in float64 (the tighter yardstick)."""
    return a.astype(np.float64) @ b.astype(np.float64).T


def gemm_bruteforce(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Triple loop with a sequential fp32 accumulator; for tiny shapes only."""
    M, K = a.shape
    N = b.shape[0]
    out = np.zeros((M, N), dtype=np.float32)
    af, bf = a.astype(np.float32), b.astype(np.float32)
    for i in range(M):
        for j in range(N):
            acc = np.float32(0)
            for k in range(K):
                acc = np.float32(acc + af[i, k] * bf[j, k])
            out[i, j] = acc
    return out


def decode_operand(raw: np.ndarray, dtype: int, mx: Optional[np.ndarray] = None) -> np.ndarray:
    """Storage bytes of A or B -> fp32 matrix [rows, K]."""
    if dtype == F16:
        return np.asarray(raw).view(np.float16).astype(np.float32)
    if dtype == BF16:
        return F.bf16_bits_to_f32(np.asarray(raw).view(np.uint16))
    if dtype == FP8_E4M3:
        return F.e4m3_decode(np.asarray(raw).view(np.uint8))
    if dtype == MXFP4:
        assert mx is not None
        return F.dequantize_mxfp4(np.asarray(raw).view(np.uint8), mx)
    raise ValueError(dtype)


def cast_output(c: np.ndarray, dtype: int) -> np.ndarray:
    """fp32 -> output storage (fp32, or uint16 bit patterns of bf16 / f16)."""
    c = np.asarray(c, dtype=np.float32)
    if dtype == F32:
        return c
    if dtype == BF16:
        return F.f32_to_bf16_bits(c)
    if dtype == F16:
        return c.astype(np.float16).view(np.uint16)
    raise ValueError(dtype)


def output_to_f32(raw: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == F32:
        return np.asarray(raw, dtype=np.float32)
    if dtype == BF16:
        return F.bf16_bits_to_f32(np.asarray(raw).view(np.uint16))
    if dtype == F16:
        return np.asarray(raw).view(np.float16).astype(np.float32)
    raise ValueError(dtype)


def gemm_epilogue(acc: np.ndarray, out_dtype: int, scale_a=None, scale_b=None,
                  bias: Optional[np.ndarray] = None) -> np.ndarray:
    v = np.asarray(acc, dtype=np.float32)
    if scale_a is not None or scale_b is not None:
        s = np.float32(1.0)
        if scale_a is not None:
            s = np.float32(s * np.float32(scale_a))
        if scale_b is not None:
            s = np.float32(s * np.float32(scale_b))
        v = (v * s).astype(np.float32)
    if bias is not None:
        v = (v + np.asarray(bias, dtype=np.float32)[None, :]).astype(np.float32)
    return cast_output(v, out_dtype)


def gemm(a_raw, b_raw, dtype_ab: int, out_dtype: int, *, mx_a=None, mx_b=None,
         scale_a=None, scale_b=None, bias=None, accumulate: str = "f32") -> np.ndarray:
    """Full path: decode -> product -> epilogue.  `accumulate` picks the fp32
    BLAS product (the reference's formula) or the float64 one rounded to fp32."""
    a = decode_operand(a_raw, dtype_ab, mx_a)
    b = decode_operand(b_raw, dtype_ab, mx_b)
    acc = gemm_f32(a, b) if accumulate == "f32" else gemm_f64(a, b).astype(np.float32)
    return gemm_epilogue(acc, out_dtype, scale_a, scale_b, bias)


def gemm_fp8(a_q, b_q, scale_a, scale_b, out_dtype=BF16, bias=None, accumulate="f32"):
    return gemm(a_q, b_q, FP8_E4M3, out_dtype, scale_a=scale_a, scale_b=scale_b, bias=bias,
                accumulate=accumulate)


def gemm_mxfp4(a_p, mx_a, b_p, mx_b, out_dtype=BF16, bias=None, accumulate="f32"):
    return gemm(a_p, b_p, MXFP4, out_dtype, mx_a=mx_a, mx_b=mx_b, bias=bias, accumulate=accumulate)


def rel_l2(got: np.ndarray, ref: np.ndarray) -> float:
    g = np.asarray(got, dtype=np.float64)
    r = np.asarray(ref, dtype=np.float64)
    den = np.linalg.norm(r)
    return float(np.linalg.norm(g - r) / den) if den > 0 else float(np.linalg.norm(g - r))
