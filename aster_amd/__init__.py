"""aster_amd: MI355X (gfx950) GEMM hot path behind the reference's config and
harness surface.  The HIP kernels live in `csrc/` and are reached through the
C-ABI of `lib/libastergemm.so` (`include/astergemm.h`)."""

from .gemm_config import (  # noqa: F401
    A, B, C, DIM_K, DIM_M, DIM_N, Cdna4GemmInstance, GemmMappingSpec, GemmSpec, LoadType,
    Operand, OperandLayout, OperandPath, WeakScaledMappedGemmInstance, make_instance,
    mfma_shape_for_mcpu, validate_gemm_config,
)
from .layout import Layout, Swizzle, tile  # noqa: F401

__all__ = [
    "A", "B", "C", "DIM_K", "DIM_M", "DIM_N", "Cdna4GemmInstance", "GemmMappingSpec", "GemmSpec",
    "LoadType", "Operand", "OperandLayout", "OperandPath", "WeakScaledMappedGemmInstance",
    "make_instance", "mfma_shape_for_mcpu", "validate_gemm_config", "Layout", "Swizzle", "tile",
]
