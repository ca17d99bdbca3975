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
_OPERAND_PATH_ID = {"lds": _capi.OPERAND_LDS, "direct_b": _capi.OPERAND_DIRECT_B,
                    "direct_b_k8": _capi.OPERAND_DIRECT_B_K8, "direct_ab": _capi.OPERAND_DIRECT_AB}
_OPERAND_PATH_NAME = {v: k for k, v in _OPERAND_PATH_ID.items()}


def config_from_instance(cfg: WeakScaledMappedGemmInstance, *, use_mapping: bool = True,
                         family: int = _capi.KERNEL_AUTO) -> _capi.Config:
    """C-ABI config for a (spec, mapping) instance.  With `use_mapping` the workgroup tile, the
    wave grid and the operand path (`direct_b`: B pre-shuffled with `shuffle_weight`) are passed
    as a request; `select_for_instance` falls back to the library's own choice when no pre-built
    kernel has that geometry and says so."""
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


@dataclass
class MappingReport:
    """How much of a GemmMappingSpec the selected pre-built kernel follows.

    `honoured`: a variant with the requested workgroup tile, wave grid and operand path exists
    for the problem and was selected.  `not_honoured`: the requested values the kernel does not
    have, each with what runs instead.  `fixed_by_kernel`: knobs that steer the reference's
    compiler (pipeline strategy, scheduler preset, peeling, barriers, load type ...) and have no
    effect on a kernel that is already built."""

    honoured: bool
    not_honoured: dict
    fixed_by_kernel: dict


_COMPILER_KNOBS = ("pipeline_strategy", "load_type", "lcm_unroll", "unroll_factor_multiplier",
                   "prologue_peeling", "epilogue_peeling", "ll_sched", "hoist_wait",
                   "set_mfma_priority", "rotate_compute_stage", "use_conservative_barriers",
                   "num_wg_per_cu")


def mapping_report(cfg: WeakScaledMappedGemmInstance, c: _capi.Config,
                   info: _capi.KernelInfo) -> MappingReport:
    spec, mapping = cfg.spec, cfg.mapping
    twg = mapping.num_tiles_per_workgroup
    want_tile = [twg[DIM_M] * spec.mfma_shape[DIM_M], twg[DIM_N] * spec.mfma_shape[DIM_N]]
    want_waves = [mapping.num_waves_per_workgroup[DIM_M], mapping.num_waves_per_workgroup[DIM_N]]
    miss = {}
    if [info.wg_tile_m, info.wg_tile_n] != want_tile:
        miss["wg_tile"] = {"requested": want_tile, "kernel": [info.wg_tile_m, info.wg_tile_n]}
    if [info.waves_m, info.waves_n] != want_waves:
        miss["waves"] = {"requested": want_waves, "kernel": [info.waves_m, info.waves_n]}
    ran_path = _OPERAND_PATH_NAME[c.operand_path]
    if mapping.operand_path.value != ran_path.replace("_k8", ""):
        miss["operand_path"] = {"requested": mapping.operand_path.value, "kernel": ran_path}
    fixed = {}
    for k in _COMPILER_KNOBS:
        if hasattr(mapping, k):
            v = getattr(mapping, k)
            fixed[k] = getattr(v, "value", v)
    return MappingReport(not miss, miss, fixed)


def select_for_instance(cfg: WeakScaledMappedGemmInstance) -> Tuple[_capi.Config, _capi.KernelInfo]:
    """Honour the instance's mapping when a variant with that geometry exists, otherwise let the
    library choose (`mapping_report` tells which happened).  A `direct_b` mapping gets a kernel
    that reads pre-shuffled B when one takes the shape -- the decode kernels in the reference's
    `shuffle_weight` order, else the stream kernels in `shuffle_weight_k8` order (fp8: step
    order; MXFP4: step order with the scale plane in lane order) (the
    returned config's `operand_path` says which; `execute_gemm_hsaco` shuffles accordingly) --
    and falls back to plain row-major B otherwise.  A `direct_ab` mapping gets the kernel that
    reads A and B both pre-shuffled with `shuffle_weight` (16-bit operands, M and N multiples of
    16), else plain row-major operands."""
    want_direct = cfg.mapping.direct_b
    if cfg.mapping.direct_a:                             # both operands pre-shuffled, no LDS
        paths = [_capi.OPERAND_DIRECT_AB]
    elif want_direct:                                    # decode kernels, then the stream kernels
        paths = [_capi.OPERAND_DIRECT_B, _capi.OPERAND_DIRECT_B_K8]
    else:
        paths = []
    for use_mapping in (True, False):
        for path in paths + [_capi.OPERAND_LDS]:
            if not use_mapping and path == _capi.OPERAND_LDS and not want_direct:
                break
            c = config_from_instance(cfg, use_mapping=use_mapping)
            c.operand_path = path
            try:
                return c, select(c)
            except _capi.AsterGemmError as e:
                if e.code != -95:
                    raise
    c = config_from_instance(cfg, use_mapping=False)
    c.operand_path = _capi.OPERAND_LDS
    return c, select(c)


def compile_gemm(cfg: WeakScaledMappedGemmInstance, output_hsaco_path: str, **kw):
    """Select the kernel for `cfg` and record it at `output_hsaco_path`.

    Returns `(path, asm)` like the reference; `asm` is a resource summary in
    `.amdgpu_metadata` spelling (`.vgpr_count`, `.lds_size`...), which is what
    harness code parses the reference's asm for.  Register budgets
    (`num_vgprs`, `num_agprs`) are accepted and ignored: the kernels are built.
    The descriptor and the summary say whether the mapping was honoured
    (`mapping_honoured`, `mapping_not_honoured`) and which of its knobs cannot
    change a pre-built kernel (`mapping_fixed_by_kernel`), so that a sweep over
    mappings can tell labels that ran the same kernel apart from real variants.
    """
    c, info = select_for_instance(cfg)
    rep = mapping_report(cfg, c, info)
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
        "operand_path": _OPERAND_PATH_NAME[c.operand_path],
        "mapping_honoured": rep.honoured,
        "mapping_not_honoured": rep.not_honoured,
        "mapping_fixed_by_kernel": rep.fixed_by_kernel,
    }
    with open(output_hsaco_path, "w") as f:
        json.dump(desc, f)
    asm = (f".amdhsa_kernel {cfg.kernel_name}\n  .name: {info.name.decode()}\n"
           f"  .vgpr_count: {info.vgprs}\n  .agpr_count: {info.agprs}\n"
           f"  .group_segment_fixed_size: {info.lds_bytes}\n"
           f"  .max_flat_workgroup_size: {info.block_x}\n"
           f"  ; mapping_honoured: {str(rep.honoured).lower()}\n")
    for k, v in rep.not_honoured.items():
        asm += f"  ; {k}: requested {v['requested']}, kernel has {v['kernel']}\n"
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
               variant: int = 0, operand_path: str = "lds", mx_a_layout: str = "rows") -> "GemmPlan":
        """`operand_path` follows GemmMappingSpec.operand_path of the reference: "lds" = B is
        plain row-major [N, ldb]; "direct_b" = B was pre-shuffled with `shuffle_weight` (the
        reference's order, read by the decode kernels; fp8 / MXFP4: `shuffle_weight_bytes`, the
        MXFP4 plane with `shuffle_scales_e8m0`); "direct_b_k8" = pre-shuffled for the stream
        kernels: 16-bit operands with `shuffle_weight_k8`, fp8 with `shuffle_weight_bytes`, MXFP4
        with `shuffle_weight_bytes` and the scale plane with `shuffle_scales_e8m0_lanes`;
        "direct_ab" = 16-bit A [M, K] and B [N, K] both pre-shuffled with `shuffle_weight`.
        `mx_a_layout` = "rows" (A's e8m0 plane [M, K/32]) or "lanes128" (in the order of
        `shuffle_scales_e8m0_lanes128` / `quantize_mxfp4_device(..., scales_layout="lanes128")`,
        read by the "direct_b_k8" MXFP4 stream kernel without a pass through LDS)."""
        c = _capi.Config()
        c.mx_a_layout = {"rows": _capi.MX_ROWS, "lanes128": _capi.MX_LANES128}[mx_a_layout]
        c.operand_path = _OPERAND_PATH_ID[operand_path]
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

    def _operands(self, dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias, workspace=None,
                  workspace_bytes=0) -> _capi.Operands:
        ops = _capi.Operands()
        ops.dA, ops.dB, ops.dC = dA, dB, dC
        ops.dScaleA, ops.dScaleB = scale_a, scale_b
        ops.dMxA, ops.dMxB = mx_a, mx_b
        ops.dBias = bias
        ops.dWorkspace, ops.workspace_bytes = workspace, workspace_bytes
        return ops

    def prepare(self) -> None:
        """Everything a first launch of this plan's kernel does on the current device apart from
        launching (function attributes, cached device facts): call before capturing launches
        of the plan into a HIP graph."""
        _capi.check(_capi.load().astergemm_prepare(ctypes.byref(self.config)))

    def workspace_bytes(self) -> int:
        """Bytes of fp32 workspace a launch of this plan needs (0 unless its rows are cut into
        K ranges); pass a buffer of that size as `workspace` to `run`, or leave it to the
        library's own buffer."""
        n = ctypes.c_size_t()
        _capi.check(_capi.load().astergemm_workspace_bytes(ctypes.byref(self.config), ctypes.byref(n)))
        return n.value

    def run(self, dA: int, dB: int, dC: int, *, scale_a: int = None, scale_b: int = None,
            mx_a: int = None, mx_b: int = None, bias: int = None, stream: int = None,
            workspace: int = None, workspace_bytes: int = 0) -> None:
        ops = self._operands(dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias, workspace,
                             workspace_bytes)
        _capi.check(_capi.load().astergemm_run(ctypes.byref(self.config), ctypes.byref(ops),
                                               ctypes.c_void_p(stream) if stream else None))

    def run_noalloc(self, dA: int, dB: int, dC: int, *, scale_a: int = None, scale_b: int = None,
                    mx_a: int = None, mx_b: int = None, bias: int = None,
                    stream: int = None) -> None:
        """`run` through the entry point that never allocates device memory: K-range partial
        sums go to the library's built-in scratch (`_capi.NOALLOC_SCRATCH_BYTES` per device)."""
        ops = self._operands(dA, dB, dC, scale_a, scale_b, mx_a, mx_b, bias)
        _capi.check(_capi.load().astergemm_run_noalloc(
            ctypes.byref(self.config), ctypes.byref(ops),
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


    def bench_graph(self, operand_sets, launches: int, replays: int) -> int:
        """`launches` launches (launch i on operand set i % len(operand_sets), sets as for
        `bench_rotate`) captured once into a HIP graph on a stream of the call's own and replayed
        `replays` times between one event pair.  Returns the total time in ns of the
        launches * replays launches: what a loop that replays a captured decode step pays."""
        arr = (_capi.Operands * len(operand_sets))()
        for i, o in enumerate(operand_sets):
            arr[i] = self._operands(o["dA"], o["dB"], o["dC"], o.get("scale_a"), o.get("scale_b"),
                                    o.get("mx_a"), o.get("mx_b"), o.get("bias"))
        total = ctypes.c_int64()
        _capi.check(_capi.load().astergemm_bench_graph(
            ctypes.byref(self.config), arr, len(operand_sets), launches, replays, ctypes.byref(total)))
        return total.value


def gemm_device(dA: int, dB: int, dC: int, M: int, N: int, K: int, dtype_ab: str = "bf16",
                dtype_c: str = "bf16", **kw) -> None:
    """One launch on caller-owned device pointers (integers)."""
    run_kw = {k: kw.pop(k) for k in ("scale_a", "scale_b", "mx_a", "mx_b", "bias", "stream")
              if k in kw}
    GemmPlan.create(M, N, K, dtype_ab, dtype_c, **kw).run(dA, dB, dC, **run_kw)


_STORAGE = {"f16": (np.dtype(np.float16), np.dtype(np.uint16)), "bf16": (np.dtype(np.uint16),),
            "fp8_e4m3": (np.dtype(np.uint8),), "mxfp4": (np.dtype(np.uint8),)}


def _row_bytes(dtype_ab: str, k: int) -> int:
    return {"f16": 2 * k, "bf16": 2 * k, "fp8_e4m3": k, "mxfp4": k // 2}[dtype_ab]


def check_host_operands(cfg: WeakScaledMappedGemmInstance, A, B, *, mx_a=None, mx_b=None,
                        bias=None) -> None:
    """Sizes and storage types of host operands against `cfg`, on the host: a kernel reads
    M*K, N*K, M*K/32, N*K/32 and N elements taken from `cfg`, so an array that is too small, or
    in another storage type, would make it read past the device allocation."""
    M, N, K = cfg.spec.gemm_size
    dt = cfg.spec.dtype_ab
    for name, arr, rows in (("A", A, M), ("B", B, N)):
        arr = np.asarray(arr)
        if arr.dtype not in _STORAGE[dt]:
            raise ValueError(f"{name} has storage type {arr.dtype}, {dt} operands are passed as "
                             f"{' or '.join(str(d) for d in _STORAGE[dt])}")
        want = rows * _row_bytes(dt, K)
        if arr.nbytes != want:
            raise ValueError(f"{name} holds {arr.nbytes} bytes, the config ({rows} rows of K={K} "
                             f"{dt} elements) needs {want}")
    if cfg.spec.scale_mode == "mx32":
        for name, arr, rows in (("mx_a", mx_a, M), ("mx_b", mx_b, N)):
            if arr is None:
                raise ValueError(f"{name} is required for MXFP4 operands")
            arr = np.asarray(arr)
            if arr.dtype != np.uint8 or arr.size != rows * (K // 32):
                raise ValueError(f"{name} must be {rows * (K // 32)} uint8 e8m0 bytes "
                                 f"([{rows}, K/32]), got {arr.size} of {arr.dtype}")
    if cfg.spec.has_bias:
        if bias is None or np.asarray(bias).size != N:
            raise ValueError(f"bias must hold N={N} values")


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
    launch, each launch between its own pair of HIP events.  B is always passed
    row-major; when the selected kernel reads pre-shuffled B (`direct_b`) the
    shuffle is done here.  Raises ValueError, before anything touches the GPU,
    when an array does not have the size or storage type `cfg` implies (the
    kernels read M*K, N*K ... elements whatever was uploaded).
    """
    check_host_operands(cfg, A, B, mx_a=mx_a, mx_b=mx_b, bias=bias)
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
    if c.operand_path != _capi.OPERAND_LDS:
        # single point of truth, as in the reference's execute_fn
        # (test_102_gemm_python_multitile_g2s_directb_cdna4.py:446-467): the caller passes B
        # row-major and the pre-shuffle happens here, in the order the kernel that runs reads
        from .kittens_helpers import (shuffle_scales_e8m0, shuffle_scales_e8m0_lanes, shuffle_weight,
                                      shuffle_weight_bytes, shuffle_weight_k8)

        if cfg.spec.dtype_ab in ("fp8_e4m3", "mxfp4"):   # byte rows in step order (+ the e8m0 plane)
            B = shuffle_weight_bytes(np.ascontiguousarray(B).reshape(N, -1).view(np.uint8))
            if mx_b is not None:   # decode kernels: step order; stream kernel: lane order
                sc_shuffle = (shuffle_scales_e8m0 if c.operand_path == _capi.OPERAND_DIRECT_B
                              else shuffle_scales_e8m0_lanes)
                mx_b = sc_shuffle(np.asarray(mx_b, dtype=np.uint8).reshape(N, K // 32))
        elif c.operand_path == _capi.OPERAND_DIRECT_AB:
            # both operands, as the reference's execute_fn does for `direct_a`
            # (test_perf_001_gemm_fp16_weak_scaled.py:252-254)
            A = shuffle_weight(np.ascontiguousarray(A).reshape(M, K))
            B = shuffle_weight(np.ascontiguousarray(B).reshape(N, K))
        else:
            shuffle = shuffle_weight if c.operand_path == _capi.OPERAND_DIRECT_B else shuffle_weight_k8
            B = shuffle(np.ascontiguousarray(B).reshape(N, K))
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


def mfma_rate(d_sample: int, sample_bytes: int, dtype_ab: str, *, target_ms: int = 50,
              stream: int = None) -> float:
    """Diagnostic: TFLOP/s the device reaches on `dtype_ab` MFMAs alone, operand registers filled
    from the sample bytes at `d_sample` (device pointer), first operand held four instructions in
    a row as in the GEMM loops.  A measured reference under the power limit, not a proven bound.
    The reference reads utilisation against the published peak only (peak_tflops_f16,
    contrib/kittens/test/bench/bench_harness.py:31-41)."""
    out = ctypes.c_double()
    _capi.check(_capi.load().astergemm_diag_mfma_rate(
        _capi.DTYPE_NAMES[dtype_ab], ctypes.c_void_p(d_sample), sample_bytes, target_ms,
        ctypes.byref(out), ctypes.c_void_p(stream) if stream else None))
    return out.value
