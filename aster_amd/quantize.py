"""Operand quantisers on the device: fp32 / bf16 / f16 -> e4m3 with a per-tensor scale, -> MXFP4.

They write the bytes the fp8 and MXFP4 GEMM kernels read.  The e4m3 rounding is the one of
the converter the reference's tests hold (f32_to_fp8_e4m3(val, fnuz=False),
test/integration/test_conversion_pack_e2e.py:91-167); the MXFP4 block layout is the operand
layout of v_mfma_scale_f32_16x16x128_f8f6f4 (include/aster/Dialect/AMDGCN/IR/Instructions/
MMA.td:792).  `*_device` functions work on device pointers the caller owns; the array
functions upload, quantise on the GPU and download with synchronous copies (tests, one-off
conversions).  There is no
CPU path.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import numpy as np

from . import _capi
from .execution import GpuBuffer


def _s(stream):
    return ctypes.c_void_p(stream) if stream else None


def _src(dtype: str) -> int:
    if dtype not in ("f32", "bf16", "f16"):
        raise ValueError(f"quantiser source must be f32, bf16 or f16, not {dtype!r}")
    return _capi.DTYPE_NAMES[dtype]


def absmax_device(d_src: int, n: int, d_absmax: int, *, src_dtype: str = "f32",
                  stream: Optional[int] = None) -> None:
    _capi.check(_capi.load().astergemm_absmax(ctypes.c_void_p(d_src), _src(src_dtype), n,
                                              ctypes.c_void_p(d_absmax), _s(stream)))


def quantize_fp8_tensor_device(d_src: int, n: int, d_dst: int, d_scale: int, *,
                               src_dtype: str = "f32", stream: Optional[int] = None) -> None:
    """d_dst[i] = e4m3(d_src[i] / scale), *d_scale = scale = absmax / 448 (1.0 for absmax 0)."""
    _capi.check(_capi.load().astergemm_quantize_fp8_tensor(
        ctypes.c_void_p(d_src), _src(src_dtype), n, ctypes.c_void_p(d_dst),
        ctypes.c_void_p(d_scale), _s(stream)))


def quantize_mxfp4_device(d_src: int, rows: int, K: int, d_packed: int, d_scales: int, *,
                          src_dtype: str = "f32", ld_src: int = 0, scales_layout: str = "rows",
                          stream: Optional[int] = None) -> None:
    """rows x K elements -> packed e2m1 [rows, K/2] and e8m0 scale bytes [rows, K/32]; with
    `scales_layout="lanes128"` the scale bytes go into the lane order of
    `kittens_helpers.shuffle_scales_e8m0_lanes128` (`mx_lanes128_bytes(rows, K)` bytes), what a
    plan with `mx_a_layout="lanes128"` reads for its activations."""
    layout = {"rows": _capi.MX_ROWS, "lanes128": _capi.MX_LANES128}[scales_layout]
    _capi.check(_capi.load().astergemm_quantize_mxfp4_ex(
        ctypes.c_void_p(d_src), _src(src_dtype), rows, K, ld_src, ctypes.c_void_p(d_packed),
        ctypes.c_void_p(d_scales), layout, _s(stream)))


def preshuffle_scales_a_device(d_mx_src: int, d_mx_dst: int, M: int, K: int, *,
                               stream: Optional[int] = None) -> None:
    """The e8m0 plane [M, K/32] of quantised activations, device to device, into the lane order
    of `kittens_helpers.shuffle_scales_e8m0_lanes128`."""
    _capi.check(_capi.load().astergemm_preshuffle_scales_a(
        M, K, ctypes.c_void_p(d_mx_src), ctypes.c_void_p(d_mx_dst), _s(stream)))


def preshuffle_device(d_src: int, d_dst: int, N: int, K: int, dtype_ab: str, operand_path: str, *,
                      d_mx_src: Optional[int] = None, d_mx_dst: Optional[int] = None,
                      stream: Optional[int] = None) -> None:
    """Weights B[N, K] row-major in device memory -> the pre-shuffled order `operand_path`
    ("direct_b" / "direct_b_k8") names for `dtype_ab`, device to device; for MXFP4 the e8m0
    plane goes from `d_mx_src` to `d_mx_dst` in the matching order (the device form of
    `kittens_helpers.shuffle_weight*` / `shuffle_scales_e8m0*`)."""
    path = {"direct_b": _capi.OPERAND_DIRECT_B, "direct_b_k8": _capi.OPERAND_DIRECT_B_K8,
            "direct_ab": _capi.OPERAND_DIRECT_AB}[operand_path]
    _capi.check(_capi.load().astergemm_preshuffle(
        _capi.DTYPE_NAMES[dtype_ab], path, N, K, ctypes.c_void_p(d_src), ctypes.c_void_p(d_dst),
        ctypes.c_void_p(d_mx_src) if d_mx_src else None,
        ctypes.c_void_p(d_mx_dst) if d_mx_dst else None, _s(stream)))


def _host_source(x: np.ndarray, dtype: Optional[str]):
    """(contiguous array, source dtype name): float32 and float16 arrays are taken as they are,
    uint16 arrays are bfloat16 bits when `dtype` says "bf16"."""
    x = np.asarray(x)
    if dtype is None:
        dtype = {np.dtype(np.float16): "f16", np.dtype(np.uint16): "bf16"}.get(x.dtype, "f32")
    want = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}[dtype]
    if dtype == "bf16" and x.dtype != np.uint16:
        raise ValueError("bf16 sources are passed as uint16 bit patterns")
    return np.ascontiguousarray(x, dtype=want), dtype


def quantize_fp8_tensor(x: np.ndarray, dtype: Optional[str] = None) -> Tuple[np.ndarray, np.float32]:
    """Array version: (e4m3 bytes of x's shape, fp32 scale)."""
    x, dtype = _host_source(x, dtype)
    src, dst, sc = GpuBuffer(max(x.nbytes, 16)), GpuBuffer(max(x.size, 4)), GpuBuffer(4)
    src.copy_from_host(x)
    quantize_fp8_tensor_device(src.ptr_value, x.size, dst.ptr_value, sc.ptr_value, src_dtype=dtype)
    q, s = np.empty(x.shape, np.uint8), np.empty(1, np.float32)
    dst.copy_to_host(q)
    sc.copy_to_host(s)
    return q, s[0]


def quantize_mxfp4(x: np.ndarray, dtype: Optional[str] = None) -> Tuple[np.ndarray, np.ndarray]:
    """Array version: x[rows, K] -> (packed [rows, K/2] uint8, scales [rows, K/32] uint8)."""
    x, dtype = _host_source(x, dtype)
    if x.ndim != 2 or x.shape[1] % 32:
        raise ValueError("quantize_mxfp4 needs a [rows, K] array with K % 32 == 0")
    rows, K = x.shape
    src, pk, sc = GpuBuffer(x.nbytes), GpuBuffer(rows * K // 2), GpuBuffer(rows * K // 32)
    src.copy_from_host(x)
    quantize_mxfp4_device(src.ptr_value, rows, K, pk.ptr_value, sc.ptr_value, src_dtype=dtype)
    packed, scales = np.empty((rows, K // 2), np.uint8), np.empty((rows, K // 32), np.uint8)
    pk.copy_to_host(packed)
    sc.copy_to_host(scales)
    return packed, scales
