"""GEMM entry points on top of the C-ABI.

Two levels:

* `compile_gemm` / `execute_gemm_hsaco` -- the harness seam every reference GEMM
  generator exposes (`compile_*(cfg, output_hsaco_path, **kw) -> (path, asm)` and
  `execute_*_hsaco(cfg, hsaco_path, num_iterations, A, B, skip_gpu_check=False)
  -> (C_flat, times_ns)`; contrib/kittens/test/
  test_102_gemm_python_multitile_g2s_directb_cdna4.py:420-467).  Nothing is
  compiled at run time here: "compiling" selects a pre-built kernel variant and
  writes a small JSON descriptor where the reference writes a code object.
* `gemm_device` / `GemmPlan` -- launches on device pointers the caller owns.

There is no CPU path: if libastergemm.so is missing, or no gfx950 device is
present, these raise.
"""

from __future__ import annotations

import ctypes
import json
from dataclasses import dataclass
from typing import List, Optional, Tuple

import numpy as np

from . import _capi
from .execution import GpuBuffer, hip_init, system_has_gpu
from .gemm_config import DIM_K, DIM_M, DIM_N, WeakScaledMappedGemmInstance

_DTYPE_ID = {"f16": _capi.F16, "bf16": _capi.BF16, "fp8_e4m3": _capi.FP8_E4M3,
             "mxfp4": _capi.MXFP4, "f32": _capi.F32}
_SCALE_ID = {"none": _capi.SCALE_NONE, "tensor": _capi.SCALE_TENSOR, "mx32": _capi.SCALE_MX32}
_OUT_NP = {"f32": np.float32, "bf16": np.uint16, "f16": np.float16}


def config_from_instance(cfg: WeakScaledMappedGemmInstance, *, use_mapping: bool = True,
                         family: int = _capi.KERNEL_AUTO) -> _capi.Config:
    """C-ABI config for a (spec, mapping) instance.  With `use_mapping` the
    workgroup tile and wave grid are passed as a request; the library falls back
    to its default variant when no pre-built kernel has that geometry."""
    spec, mapping = cfg.spec, cfg.mapping
    M, N, K = spec.gemm_size
    c = _capi.Config()
    c.M, c.N, c.K = M, N, K
    c.dtype_ab = _DTYPE_ID[spec.dtype_ab]
    c.dtype_c = _DTYPE_ID[spec.dtype_c]
    c.scale_mode = _SCALE_ID[spec.scale_mode]
    c.has_bias = int(spec.has_bias)
    c.family = family
    if use_mapping:
        twg = mapping.num_tiles_per_workgroup
        c.wg_tile_m = twg[DIM_M] * spec.mfma_shape[DIM_M]
        c.wg_tile_n = twg[DIM_N] * spec.mfma_shape[DIM_N]
        c.waves_m = mapping.num_waves_per_workgroup[DIM_M]
        c.waves_n = mapping.num_waves_per_workgroup[DIM_N]
    return c


def select(c: _capi.Config) -> _capi.KernelInfo:
    info = _capi.KernelInfo()
    _capi.check(_capi.load().astergemm_select(ctypes.byref(c), ctypes.byref(info)))
    return info


def select_for_instance(cfg: WeakScaledMappedGemmInstance) -> Tuple[_capi.Config, _capi.KernelInfo]:
    """Honour the instance's mapping when a variant with that geometry exists,
    otherwise let the library choose."""
    c = config_from_instance(cfg, use_mapping=True)
    try:
        return c, select(c)
    except _capi.AsterGemmError as e:
        if e.code != -95:
            raise
    c = config_from_instance(cfg, use_mapping=False)
    return c, select(c)


def compile_gemm(cfg: WeakScaledMappedGemmInstance, output_hsaco_path: str, **kw):
    """Select the kernel for `cfg` and record it at `output_hsaco_path`.

    Returns `(path, asm)` like the reference; `asm` is a resource summary in
    `.amdgpu_metadata` spelling (`.vgpr_count`, `.lds_size`...), which is what
    harness code parses the reference's asm for.  Register budgets
    (`num_vgprs`, `num_agprs`) are accepted and ignored: the kernels are built.
    """
    c, info = select_for_instance(cfg)
    desc = {
        "format": "astergemm-descriptor-v1",
        "label": cfg.label,
        "kernel": info.name.decode(),
        "variant": info.variant,
        "grid": info.grid_x,
        "block": info.block_x,
        "lds_bytes": info.lds_bytes,
        "vgprs": info.vgprs,
        "wg_tile": [info.wg_tile_m, info.wg_tile_n, info.wg_tile_k],
        "waves": [info.waves_m, info.waves_n],
    }
    with open(output_hsaco_path, "w") as f:
        json.dump(desc, f)
    asm = (f".amdhsa_kernel {cfg.kernel_name}\n  .name: {info.name.decode()}\n"
           f"  .vgpr_count: {info.vgprs}\n  .agpr_count: {info.agprs}\n"
           f"  .group_segment_fixed_size: {info.lds_bytes}\n"
           f"  .max_flat_workgroup_size: {info.block_x}\n")
    return output_hsaco_path, asm


def _read_descriptor(path: str) -> dict:
    with open(path) as f:
        desc = json.load(f)
    if desc.get("format") != "astergemm-descriptor-v1":
        raise ValueError(f"{path} is not an astergemm kernel descriptor")
    return desc


@dataclass
class GemmPlan:
    """A selected kernel plus its C-ABI config; launches on device pointers."""

    config: _capi.Config
    info: _capi.KernelInfo

    @classmethod
    def create(cls, M: int, N: int, K: int, dtype_ab: str = "bf16", dtype_c: str = "bf16", *,
               scale_mode: Optional[str] = None, has_bias: bool = False, lda: int = 0,
               ldb: int = 0, ldc: int = 0, family: int = _capi.KERNEL_AUTO, wg_tile=(0, 0),
               variant: int = 0, operand_path: str = "lds") -> "GemmPlan":
        """`operand_path` follows GemmMappingSpec.operand_path of the reference: "lds" = B is
        plain row-major [N, ldb]; "direct_b" = B was pre-shuffled with `shuffle_weight`."""
        c = _capi.Config()
        c.operand_path = {"lds": _capi.OPERAND_LDS, "direct_b": _capi.OPERAND_DIRECT_B}[operand_path]
        c.M, c.N, c.K = M, N, K
        c.lda, c.ldb, c.ldc = lda, ldb, ldc
        c.dtype_ab, c.dtype_c = _DTYPE_ID[dtype_ab], _DTYPE_ID[dtype_c]
        if scale_mode is None:
            scale_mode = {"fp8_e4m3": "tensor", "mxfp4": "mx32"}.get(dtype_ab, "none")
        c.scale_mode = _SCALE_ID[scale_mode]
        c.has_bias = int(has_bias)
        c.family = family
        c.wg_tile_m, c.wg_tile_n = wg_tile
        c.variant = variant
        return cls(c, select(c))

    def _operands(self, dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias) -> _capi.Operands:
        ops = _capi.Operands()
        ops.dA, ops.dB, ops.dC = dA, dB, dC
        ops.dScaleA, ops.dScaleB = scale_a, scale_b
        ops.dMxA, ops.dMxB = mx_a, mx_b
        ops.dBias = bias
        return ops

    def run(self, dA: int, dB: int, dC: int, *, scale_a: int = None, scale_b: int = None,
            mx_a: int = None, mx_b: int = None, bias: int = None, stream: int = None) -> None:
        ops = self._operands(dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias)
        _capi.check(_capi.load().astergemm_run(ctypes.byref(self.config), ctypes.byref(ops),
                                               ctypes.c_void_p(stream) if stream else None))

    def bench(self, dA: int, dB: int, dC: int, iters: int, *, scale_a: int = None,
              scale_b: int = None, mx_a: int = None, mx_b: int = None, bias: int = None,
              flush_bytes: int = 0, stream: int = None) -> List[int]:
        ops = self._operands(dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias)
        times = (ctypes.c_int64 * iters)()
        _capi.check(_capi.load().astergemm_bench(
            ctypes.byref(self.config), ctypes.byref(ops), iters, times, flush_bytes,
            ctypes.c_void_p(stream) if stream else None))
        return list(times)


    def tune(self, dA: int, dB: int, dC: int, iters: int = 10, *, scale_a: int = None,
             scale_b: int = None, mx_a: int = None, mx_b: int = None, bias: int = None,
             stream: int = None) -> "GemmPlan":
        """Times every variant that can run this plan's problem on the given operands and
        returns a plan pinned to the fastest (`plan.tuned_ns` = its time per launch).  dC is
        overwritten by every candidate."""
        ops = self._operands(dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias)
        cfg = _capi.Config.from_buffer_copy(self.config)
        cfg.variant = 0
        best, ns = ctypes.c_int(), ctypes.c_int64()
        _capi.check(_capi.load().astergemm_tune(
            ctypes.byref(cfg), ctypes.byref(ops), iters, ctypes.byref(best), ctypes.byref(ns),
            ctypes.c_void_p(stream) if stream else None))
        cfg.variant = best.value
        plan = GemmPlan(cfg, select(cfg))
        plan.tuned_ns = ns.value
        return plan

    def bench_rotate(self, operand_sets, iters: int, stream: int = None) -> int:
        """`iters` back-to-back launches between one event pair, launch i on operand set
        i % len(operand_sets); each set is a dict with dA, dB, dC and optional scale_a,
        scale_b, mx_a, mx_b, bias device pointers.  Returns the total time in ns."""
        arr = (_capi.Operands * len(operand_sets))()
        for i, o in enumerate(operand_sets):
            arr[i] = self._operands(o["dA"], o["dB"], o["dC"], o.get("scale_a"), o.get("scale_b"),
                                    o.get("mx_a"), o.get("mx_b"), o.get("bias"))
        total = ctypes.c_int64()
        _capi.check(_capi.load().astergemm_bench_rotate(
            ctypes.byref(self.config), arr, len(operand_sets), iters, ctypes.byref(total),
            ctypes.c_void_p(stream) if stream else None))
        return total.value


def gemm_device(dA: int, dB: int, dC: int, M: int, N: int, K: int, dtype_ab: str = "bf16",
                dtype_c: str = "bf16", **kw) -> None:
    """One launch on caller-owned device pointers (integers)."""
    run_kw = {k: kw.pop(k) for k in ("scale_a", "scale_b", "mx_a", "mx_b", "bias", "stream")
              if k in kw}
    GemmPlan.create(M, N, K, dtype_ab, dtype_c, **kw).run(dA, dB, dC, **run_kw)


def execute_gemm_hsaco(cfg: WeakScaledMappedGemmInstance, hsaco_path: str, num_iterations: int,
                       A: np.ndarray, B: np.ndarray, skip_gpu_check: bool = False, *,
                       scale_a: Optional[float] = None, scale_b: Optional[float] = None,
                       mx_a: Optional[np.ndarray] = None, mx_b: Optional[np.ndarray] = None,
                       bias: Optional[np.ndarray] = None, flush_bytes: int = 0):
    """Run the kernel recorded by `compile_gemm` on host arrays.

    A is [M, K] and B is [N, K] in the storage type of `cfg.spec.dtype_ab`
    (np.float16, or np.uint16 bit patterns for bf16, np.uint8 for fp8 / packed
    fp4).  Returns `(C_flat, times_ns)`: C flattened in `cfg.spec.dtype_c`
    storage (float32; uint16 bit patterns for bf16; float16), one time per
    launch, each launch between its own pair of HIP events.  Unlike the
    reference's direct-B kernels no host pre-shuffle of B is needed.
    """
    mcpu = getattr(cfg.mapping, "mcpu", "gfx950")
    if not skip_gpu_check and not system_has_gpu("gfx950"):
        import pytest

        pytest.skip(f"GPU {mcpu} not available, skip execution")
    desc = _read_descriptor(hsaco_path)
    hip_init()
    c, info = select_for_instance(cfg)
    if info.name.decode() != desc["kernel"]:
        raise RuntimeError(f"descriptor names kernel {desc['kernel']!r} but config selects "
                           f"{info.name.decode()!r}")
    M, N, K = cfg.spec.gemm_size
    out_np = _OUT_NP[cfg.spec.dtype_c]
    C_host = np.zeros(M * N, dtype=out_np)

    def up(arr, dtype=None):
        if arr is None:
            return None
        a = np.ascontiguousarray(arr if dtype is None else np.asarray(arr, dtype=dtype))
        buf = GpuBuffer(a.nbytes)
        buf.copy_from_host(a)
        return buf

    bufs = {"A": up(A), "B": up(B), "C": GpuBuffer(C_host.nbytes)}
    if cfg.spec.scale_mode == "tensor":
        bufs["sa"] = up(np.array([1.0 if scale_a is None else scale_a], dtype=np.float32))
        bufs["sb"] = up(np.array([1.0 if scale_b is None else scale_b], dtype=np.float32))
    if cfg.spec.scale_mode == "mx32":
        bufs["mxa"], bufs["mxb"] = up(mx_a, np.uint8), up(mx_b, np.uint8)
    if cfg.spec.has_bias:
        bufs["bias"] = up(bias, np.float32)
    ptr = lambda k: bufs[k].ptr_value if bufs.get(k) is not None else None
    plan = GemmPlan(c, info)
    try:
        kw = dict(scale_a=ptr("sa"), scale_b=ptr("sb"), mx_a=ptr("mxa"), mx_b=ptr("mxb"),
                  bias=ptr("bias"))
        # First launch, then the copy back (the reference copies after iteration 0).
        times = plan.bench(ptr("A"), ptr("B"), ptr("C"), 1, flush_bytes=flush_bytes, **kw)
        bufs["C"].copy_to_host(C_host)
        if num_iterations > 1:
            times += plan.bench(ptr("A"), ptr("B"), ptr("C"), num_iterations - 1,
                                flush_bytes=flush_bytes, **kw)
    finally:
        for b in bufs.values():
            if b is not None:
                b.free()
    return C_host, times


def mfma_ceiling(d_sample: int, sample_bytes: int, dtype_ab: str, *, target_ms: int = 50,
                 stream: int = None) -> float:
    """TFLOP/s the device sustains on `dtype_ab` MFMAs alone, operand registers filled from the
    sample bytes at `d_sample` (device pointer): the rate no GEMM on such values can exceed
    under the power limit.  The reference reads utilisation against the published peak only
    (peak_tflops_f16, contrib/kittens/test/bench/bench_harness.py:31-41)."""
    out = ctypes.c_double()
    _capi.check(_capi.load().astergemm_mfma_ceiling(
        _capi.DTYPE_NAMES[dtype_ab], ctypes.c_void_p(d_sample), sample_bytes, target_ms,
        ctypes.byref(out), ctypes.c_void_p(stream) if stream else None))
    return out.value
