"""Weight artefact files: B[N, K] on disk in the bytes the kernels stream.

The reference prepares weights on every call: `execute_fn` pre-shuffles B with
`shuffle_weight` when the mapping says direct_b
(contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:440-467,
contrib/kittens/test/kittens_helpers.py:90-119) and its fp8 tests convert on the host
(test/integration/test_conversion_pack_e2e.py:91-167).  An artefact is that preparation done
once: a 128-byte header (`astergemm_weight_header`: magic, version, dtype, layout, N, K,
section offsets, CRC-32 of each section, the fp8 tensor scale) followed by the payload and,
for MXFP4, the e8m0 scale plane.  Loading is one read and one upload; nothing is converted
or permuted.  Header logic and checksums live in the C library (`astergemm_weight_*`); this
module does the file I/O, the one-off packing and the device side.

fp8 and MXFP4 packing runs on the GPU quantisers (there is no CPU quantiser in the product).
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import numpy as np

from . import _capi
from .execution import GpuBuffer
from .gemm import GemmPlan
from .kittens_helpers import (shuffle_scales_e8m0, shuffle_scales_e8m0_lanes, shuffle_weight,
                              shuffle_weight_bytes, shuffle_weight_k8)

_LAYOUT_ID = {"lds": _capi.OPERAND_LDS, "direct_b": _capi.OPERAND_DIRECT_B,
              "direct_b_k8": _capi.OPERAND_DIRECT_B_K8}
_LAYOUT_NAME = {v: k for k, v in _LAYOUT_ID.items()}
_DTYPE_NAME = {v: k for k, v in _capi.DTYPE_NAMES.items()}


def _bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)


class WeightArtifact:
    """Header + payload (+ scale plane) of one weight matrix, in host memory or mapped."""

    def __init__(self, header: _capi.WeightHeader, payload: np.ndarray,
                 scales: Optional[np.ndarray] = None) -> None:
        self.header, self.payload, self.scales = header, payload, scales

    # ---- description -------------------------------------------------------------------
    @property
    def dtype(self) -> str:
        return _DTYPE_NAME[self.header.dtype]

    @property
    def layout(self) -> str:
        return _LAYOUT_NAME[self.header.layout]

    @property
    def shape(self):
        return int(self.header.N), int(self.header.K)

    @property
    def tensor_scale(self) -> float:
        return float(self.header.tensor_scale)

    # ---- construction ------------------------------------------------------------------
    @classmethod
    def from_storage(cls, bits: np.ndarray, dtype: str, N: int, K: int, *, layout: str = "lds",
                     scales: Optional[np.ndarray] = None, tensor_scale: float = 1.0
                     ) -> "WeightArtifact":
        """`bits` is the matrix as a kernel reads it: [N, K] float16 / uint16 (bf16 bits) /
        uint8 (e4m3), or [N, K/2] uint8 nibbles with `scales` [N, K/32] for MXFP4.  For
        layout "direct_b" the bits must already be in `shuffle_weight` order (16-bit types) or
        `shuffle_weight_bytes` order (fp8, MXFP4; the MXFP4 plane in `shuffle_scales_e8m0` order),
        for "direct_b_k8" in `shuffle_weight_k8` order (16-bit types) or `shuffle_weight_bytes`
        order (fp8; MXFP4, with the plane in `shuffle_scales_e8m0_lanes` order)."""
        h = _capi.WeightHeader()
        _capi.check(_capi.load().astergemm_weight_header_init(
            ctypes.byref(h), _capi.DTYPE_NAMES[dtype], _LAYOUT_ID[layout], N, K,
            ctypes.c_float(tensor_scale)))
        payload = np.ascontiguousarray(bits).reshape(-1).view(np.uint8)
        if payload.nbytes != h.payload_bytes:
            raise ValueError(f"payload has {payload.nbytes} bytes, {dtype} [{N}, {K}] needs "
                             f"{h.payload_bytes}")
        if h.scales_bytes:
            if scales is None:
                raise ValueError("MXFP4 needs the e8m0 scale plane")
            scales = np.ascontiguousarray(scales, dtype=np.uint8).reshape(-1)
            if scales.nbytes != h.scales_bytes:
                raise ValueError(f"scale plane has {scales.nbytes} bytes, needs {h.scales_bytes}")
        elif scales is not None:
            raise ValueError(f"{dtype} takes no scale plane")
        lib = _capi.load()
        h.payload_crc32 = lib.astergemm_weight_crc32(payload.ctypes.data, payload.nbytes)
        if h.scales_bytes:
            h.scales_crc32 = lib.astergemm_weight_crc32(scales.ctypes.data, scales.nbytes)
        return cls(h, payload, scales)

    @classmethod
    def from_f32(cls, w: np.ndarray, dtype: str, *, layout: str = "lds") -> "WeightArtifact":
        """Pack an fp32 matrix W[N, K]: f16 / bf16 are rounded on the host (and pre-shuffled
        for the layouts "direct_b" and "direct_b_k8"); fp8 and MXFP4 go through the GPU quantisers."""
        w = np.ascontiguousarray(w, dtype=np.float32)
        if w.ndim != 2:
            raise ValueError("from_f32: W must be [N, K]")
        N, K = w.shape
        if dtype in ("f16", "bf16"):
            bits = w.astype(np.float16).view(np.uint16) if dtype == "f16" else _bf16_bits(w)
            if layout == "direct_b":
                bits = shuffle_weight(bits)
            elif layout == "direct_b_k8":
                bits = shuffle_weight_k8(bits)
            return cls.from_storage(bits, dtype, N, K, layout=layout)
        from . import quantize as Q
        if dtype == "fp8_e4m3":
            q, s = Q.quantize_fp8_tensor(w)
            if layout in ("direct_b", "direct_b_k8"):   # step order for both kernel sets
                q = shuffle_weight_bytes(np.asarray(q).reshape(N, K).view(np.uint8))
            return cls.from_storage(q, dtype, N, K, layout=layout, tensor_scale=float(s))
        if dtype == "mxfp4":
            p, s = Q.quantize_mxfp4(w)
            if layout in ("direct_b", "direct_b_k8"):   # decode kernels / stream kernel
                p = shuffle_weight_bytes(np.asarray(p).reshape(N, K // 2).view(np.uint8))
                sc_shuffle = shuffle_scales_e8m0 if layout == "direct_b" else shuffle_scales_e8m0_lanes
                s = sc_shuffle(np.asarray(s).reshape(N, K // 32))
            return cls.from_storage(p, dtype, N, K, layout=layout, scales=s)
        raise ValueError(f"from_f32: unknown dtype {dtype!r}")

    # ---- file I/O ------------------------------------------------------------------------
    def save(self, path: str) -> None:
        h = self.header
        tmp = str(path) + ".tmp"
        with open(tmp, "wb") as f:
            f.write(bytes(h))
            f.write(b"\0" * (h.payload_offset - ctypes.sizeof(h)))
            f.write(self.payload.tobytes() if not isinstance(self.payload, np.memmap)
                    else bytes(self.payload))
            if h.scales_bytes:
                f.write(b"\0" * (h.scales_offset - h.payload_offset - h.payload_bytes))
                f.write(self.scales.tobytes())
        os.replace(tmp, path)

    @classmethod
    def load(cls, path: str, *, verify: bool = True) -> "WeightArtifact":
        """Maps the file (read-only); `verify` also checks both checksums, which reads it all."""
        size = os.path.getsize(path)
        if size < ctypes.sizeof(_capi.WeightHeader):
            raise _capi.AsterGemmError(-22, "astergemm_weight: file shorter than the header")
        image = np.memmap(path, dtype=np.uint8, mode="r")
        lib = _capi.load()
        h = _capi.WeightHeader()
        head = np.array(image[:ctypes.sizeof(h)])
        # the header check needs the file size, not the bytes behind the header
        _capi.check(lib.astergemm_weight_header_check(head.ctypes.data, size, ctypes.byref(h)))
        payload = image[h.payload_offset:h.payload_offset + h.payload_bytes]
        scales = image[h.scales_offset:h.scales_offset + h.scales_bytes] if h.scales_bytes else None
        if verify:
            for name, sec, want in (("payload", payload, h.payload_crc32),
                                    ("scale plane", scales, h.scales_crc32)):
                if sec is None:
                    continue
                buf = np.ascontiguousarray(sec)
                if lib.astergemm_weight_crc32(buf.ctypes.data, buf.nbytes) != want:
                    raise _capi.AsterGemmError(-22, f"astergemm_weight: {name} checksum mismatch")
        return cls(h, payload, scales)

    # ---- device side ---------------------------------------------------------------------
    def to_device(self) -> "DeviceWeight":
        return DeviceWeight(self)


class DeviceWeight:
    """An artefact resident in HBM, with the plans that multiply activations by it."""

    def __init__(self, art: WeightArtifact) -> None:
        self.header = art.header
        self._b = GpuBuffer(art.payload.nbytes)
        self._b.copy_from_host(np.ascontiguousarray(art.payload))
        self._mx = None
        if art.scales is not None:
            self._mx = GpuBuffer(art.scales.nbytes)
            self._mx.copy_from_host(np.ascontiguousarray(art.scales))
        self._scale = None
        if art.header.scale_mode == _capi.SCALE_TENSOR:
            self._scale = GpuBuffer(4)
            self._scale.copy_from_host(np.array([art.header.tensor_scale], np.float32))
        self._plans = {}

    @property
    def weight_ptr(self) -> int:
        return self._b.ptr_value

    def plan(self, M: int, dtype_c: str = "bf16", has_bias: bool = False) -> GemmPlan:
        key = (M, dtype_c, has_bias)
        if key not in self._plans:
            c = _capi.Config()
            _capi.check(_capi.load().astergemm_weight_config(
                ctypes.byref(self.header), M, _capi.DTYPE_NAMES[dtype_c], ctypes.byref(c)))
            c.has_bias = int(has_bias)
            from .gemm import select
            self._plans[key] = GemmPlan(c, select(c))
        return self._plans[key]

    def run(self, d_x: int, d_out: int, M: int, dtype_c: str = "bf16", *, scale_x: int = None,
            mx_x: int = None, bias: int = None, stream: int = None) -> None:
        """out[M, N] = x[M, K] @ W^T on device pointers; `scale_x` (fp8) / `mx_x` (MXFP4) are
        the activation's scale operands."""
        self.plan(M, dtype_c, bias is not None).run(
            d_x, self._b.ptr_value, d_out, scale_a=scale_x,
            scale_b=self._scale.ptr_value if self._scale else None, mx_a=mx_x,
            mx_b=self._mx.ptr_value if self._mx else None, bias=bias, stream=stream)

    def free(self) -> None:
        for b in (self._b, self._mx, self._scale):
            if b is not None:
                b.free()
