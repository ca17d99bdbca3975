"""ctypes binding of libastergemm.so (the C-ABI declared in include/astergemm.h).

The reference binds its native runtime with nanobind
(`aster._mlir_libs._runtime_module`, python/lib/RuntimeModule.cpp:140-418);
nanobind is not part of this toolchain, so the same functions are reached
through ctypes.  There is no fallback: if the shared library is missing or a
call fails, an exception is raised.
"""

from __future__ import annotations

import ctypes as C
import importlib.util
import os
import sys
from typing import Optional

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libastergemm.so")

# astergemm_dtype
F16, BF16, FP8_E4M3, MXFP4, F32 = 0, 1, 2, 3, 4
# astergemm_scale_mode
SCALE_NONE, SCALE_TENSOR, SCALE_MX32 = 0, 1, 2
# astergemm_kernel_family
KERNEL_AUTO, KERNEL_TILE, KERNEL_SKINNY = 0, 1, 2
OPERAND_LDS, OPERAND_DIRECT_B, OPERAND_DIRECT_B_K8, OPERAND_DIRECT_AB = 0, 1, 2, 3
# astergemm_mx_layout
MX_ROWS, MX_LANES128 = 0, 1
ABI_VERSION = 3
NOALLOC_SCRATCH_BYTES = 16 << 20

DTYPE_NAMES = {"f16": F16, "bf16": BF16, "fp8_e4m3": FP8_E4M3, "mxfp4": MXFP4, "f32": F32}


class AsterGemmError(RuntimeError):
    """A libastergemm call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[{code}] {message}")
        self.code = code


class Config(C.Structure):
    _fields_ = [
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
        ("dtype_ab", C.c_int32), ("dtype_c", C.c_int32),
        ("scale_mode", C.c_int32), ("has_bias", C.c_int32),
        ("family", C.c_int32),
        ("wg_tile_m", C.c_int32), ("wg_tile_n", C.c_int32),
        ("waves_m", C.c_int32), ("waves_n", C.c_int32),
        ("variant", C.c_int32),
        ("operand_path", C.c_int32),
        ("mx_a_layout", C.c_int32),
        ("reserved", C.c_int32 * 4),
    ]


class KernelInfo(C.Structure):
    _fields_ = [
        ("variant", C.c_int32), ("family", C.c_int32),
        ("grid_x", C.c_int32), ("block_x", C.c_int32),
        ("lds_bytes", C.c_int32), ("vgprs", C.c_int32), ("agprs", C.c_int32),
        ("wg_tile_m", C.c_int32), ("wg_tile_n", C.c_int32), ("wg_tile_k", C.c_int32),
        ("waves_m", C.c_int32), ("waves_n", C.c_int32),
        ("pipeline_stages", C.c_int32),
        ("flops", C.c_int64), ("bytes", C.c_int64),
        ("name", C.c_char * 64),
    ]


class Operands(C.Structure):
    _fields_ = [
        ("dA", C.c_void_p), ("dB", C.c_void_p), ("dC", C.c_void_p),
        ("dScaleA", C.c_void_p), ("dScaleB", C.c_void_p),
        ("dMxA", C.c_void_p), ("dMxB", C.c_void_p),
        ("dBias", C.c_void_p),
        ("dWorkspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
    ]


class DeviceProps(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128), ("gcn_arch_name", C.c_char * 64),
        ("warp_size", C.c_int32), ("lds_per_cu", C.c_int32),
        ("regs_per_multiprocessor", C.c_int32), ("multiprocessor_count", C.c_int32),
        ("max_threads_per_block", C.c_int32), ("max_threads_per_multiprocessor", C.c_int32),
        ("asic_revision", C.c_int32), ("cluster_launch", C.c_int32),
        ("total_global_mem", C.c_int64),
        ("clock_rate_khz", C.c_int32), ("l2_cache_bytes", C.c_int32),
    ]


class WeightHeader(C.Structure):
    """astergemm_weight_header: the 128-byte header of a weight artefact file."""
    _fields_ = [
        ("magic", C.c_char * 8),
        ("version", C.c_uint32), ("header_bytes", C.c_uint32),
        ("dtype", C.c_uint32), ("layout", C.c_uint32), ("scale_mode", C.c_uint32),
        ("tensor_scale", C.c_float),
        ("N", C.c_int64), ("K", C.c_int64),
        ("payload_offset", C.c_int64), ("payload_bytes", C.c_int64),
        ("scales_offset", C.c_int64), ("scales_bytes", C.c_int64),
        ("payload_crc32", C.c_uint32), ("scales_crc32", C.c_uint32),
        ("reserved", C.c_uint8 * 40),
    ]


# name -> (restype, argtypes); every symbol include/astergemm.h declares.
_P = C.c_void_p
SIGNATURES = {
    "astergemm_abi_version": (C.c_int, []),
    "astergemm_last_error": (C.c_char_p, []),
    "astergemm_select": (C.c_int, [C.POINTER(Config), C.POINTER(KernelInfo)]),
    "astergemm_variant_count": (C.c_int, []),
    "astergemm_variant_info": (C.c_int, [C.c_int, C.POINTER(Config), C.POINTER(KernelInfo)]),
    "astergemm_run": (C.c_int, [C.POINTER(Config), C.POINTER(Operands), _P]),
    "astergemm_run_noalloc": (C.c_int, [C.POINTER(Config), C.POINTER(Operands), _P]),
    "astergemm_prepare": (C.c_int, [C.POINTER(Config)]),
    "astergemm_workspace_bytes": (C.c_int, [C.POINTER(Config), C.POINTER(C.c_size_t)]),
    "astergemm_bench_rotate": (C.c_int, [C.POINTER(Config), C.POINTER(Operands), C.c_int, C.c_int,
                                         C.POINTER(C.c_int64), C.c_void_p]),
    "astergemm_bench_graph": (C.c_int, [C.POINTER(Config), C.POINTER(Operands), C.c_int, C.c_int,
                                        C.c_int, C.POINTER(C.c_int64)]),
    "astergemm_bench": (C.c_int, [C.POINTER(Config), C.POINTER(Operands), C.c_int,
                                  C.POINTER(C.c_int64), C.c_int64, _P]),
    "astergemm_tune": (C.c_int, [C.POINTER(Config), C.POINTER(Operands), C.c_int, C.POINTER(C.c_int),
                                 C.POINTER(C.c_int64), _P]),
    "astergemm_diag_mfma_rate": (C.c_int, [C.c_int, _P, C.c_int64, C.c_int, C.POINTER(C.c_double), _P]),
    "astergemm_shuffle_weight_16": (C.c_int, [_P, _P, C.c_int64, C.c_int64]),
    "astergemm_shuffle_weight_k8_16": (C.c_int, [_P, _P, C.c_int64, C.c_int64]),
    "astergemm_shuffle_weight_8": (C.c_int, [_P, _P, C.c_int64, C.c_int64]),
    "astergemm_shuffle_scales_e8m0": (C.c_int, [_P, _P, C.c_int64, C.c_int64]),
    "astergemm_shuffle_scales_e8m0_lanes": (C.c_int, [_P, _P, C.c_int64, C.c_int64]),
    "astergemm_mx_lanes128_bytes": (C.c_int64, [C.c_int64, C.c_int64]),
    "astergemm_shuffle_scales_e8m0_lanes128": (C.c_int, [_P, _P, C.c_int64, C.c_int64]),
    "astergemm_preshuffle_scales_a": (C.c_int, [C.c_int64, C.c_int64, _P, _P, _P]),
    "astergemm_quantize_mxfp4_ex": (C.c_int, [_P, C.c_int, C.c_int64, C.c_int64, C.c_int64, _P, _P,
                                              C.c_int, _P]),
    "astergemm_preshuffle": (C.c_int, [C.c_int, C.c_int, C.c_int64, C.c_int64, _P, _P, _P, _P, _P]),
    "astergemm_weight_crc32": (C.c_uint32, [_P, C.c_size_t]),
    "astergemm_weight_header_init": (C.c_int, [C.POINTER(WeightHeader), C.c_int, C.c_int, C.c_int64,
                                               C.c_int64, C.c_float]),
    "astergemm_weight_header_check": (C.c_int, [_P, C.c_size_t, C.POINTER(WeightHeader)]),
    "astergemm_weight_verify": (C.c_int, [_P, C.c_size_t]),
    "astergemm_weight_config": (C.c_int, [C.POINTER(WeightHeader), C.c_int64, C.c_int,
                                          C.POINTER(Config)]),
    "astergemm_absmax": (C.c_int, [_P, C.c_int, C.c_int64, _P, _P]),
    "astergemm_quantize_fp8_tensor": (C.c_int, [_P, C.c_int, C.c_int64, _P, _P, _P]),
    "astergemm_quantize_mxfp4": (C.c_int, [_P, C.c_int, C.c_int64, C.c_int64, C.c_int64, _P, _P, _P]),
    "aster_rt_init": (C.c_int, []),
    "aster_rt_peek_at_last_error": (C.c_int, []),
    "aster_rt_clear_last_error": (C.c_int, []),
    "aster_rt_get_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "aster_rt_set_device": (C.c_int, [C.c_int]),
    "aster_rt_get_device": (C.c_int, [C.POINTER(C.c_int)]),
    "aster_rt_device_reset": (C.c_int, []),
    "aster_rt_device_synchronize": (C.c_int, []),
    "aster_rt_get_device_props": (C.c_int, [C.c_int, C.POINTER(DeviceProps)]),
    "aster_rt_malloc": (C.c_int, [C.POINTER(_P), C.c_size_t]),
    "aster_rt_free": (C.c_int, [_P]),
    "aster_rt_memcpy_h2d": (C.c_int, [_P, _P, C.c_size_t]),
    "aster_rt_memcpy_d2h": (C.c_int, [_P, _P, C.c_size_t]),
    "aster_rt_memcpy_d2d": (C.c_int, [_P, _P, C.c_size_t]),
    "aster_rt_memset": (C.c_int, [_P, C.c_int, C.c_size_t]),
    "aster_rt_module_load_data": (C.c_int, [_P, C.c_size_t, C.POINTER(_P)]),
    "aster_rt_module_get_function": (C.c_int, [_P, C.c_char_p, C.POINTER(_P)]),
    "aster_rt_module_unload": (C.c_int, [_P]),
    "aster_rt_module_launch_kernel": (C.c_int, [_P] + [C.c_uint] * 7 + [_P, C.POINTER(_P)]),
    "aster_rt_function_free": (C.c_int, [_P]),
    "aster_rt_module_launch_kernel_ex": (C.c_int, [_P] + [C.c_uint] * 10 + [_P, C.POINTER(_P)]),
    "aster_rt_event_create": (C.c_int, [C.POINTER(_P)]),
    "aster_rt_event_destroy": (C.c_int, [_P]),
    "aster_rt_event_record": (C.c_int, [_P, _P]),
    "aster_rt_event_synchronize": (C.c_int, [_P]),
    "aster_rt_event_elapsed_ms": (C.c_int, [_P, _P, C.POINTER(C.c_float)]),
    "aster_rt_stream_create": (C.c_int, [C.POINTER(_P)]),
    "aster_rt_stream_destroy": (C.c_int, [_P]),
    "aster_rt_stream_synchronize": (C.c_int, [_P]),
}

_lib: Optional[C.CDLL] = None


def library_path() -> str:
    return _LIB_PATH


def _bind_one_hip_runtime() -> None:
    """PyTorch's ROCm wheels carry a HIP runtime of their own (torch/lib/libamdhip64.so,
    SONAME libamdhip64.so.7) and ask for it under the file name, not the SONAME.  Loaded after
    the system's copy, which libastergemm.so would pull in when it comes first, the process holds
    two runtimes, and the one that initialises second reports that it finds no device.  When
    PyTorch is installed and not yet imported, its copy is therefore loaded first: the
    library's request for libamdhip64.so.7 then resolves to it, and so does PyTorch's later.
    A process without PyTorch keeps the system's runtime."""
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.origin:
        return
    path = os.path.join(os.path.dirname(spec.origin), "lib", "libamdhip64.so")
    if os.path.exists(path):
        C.CDLL(path, mode=C.RTLD_GLOBAL)


def load() -> C.CDLL:
    """Load libastergemm.so and attach the prototypes. Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    _bind_one_hip_runtime()
    if not os.path.exists(_LIB_PATH):
        raise FileNotFoundError(
            f"{_LIB_PATH} is not built; run `python -m aster_amd.build` "
            "(needs hipcc; cross-compiles for gfx950 without a GPU)"
        )
    lib = C.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error() -> str:
    msg = load().astergemm_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc: int) -> None:
    if rc != 0:
        raise AsterGemmError(rc, last_error())
