"""GEMM problem, GPU mapping and validated (problem, mapping) instances.

Host-side mirror of the reference's config surface
(contrib/kittens/gemm_config.py): `GemmSpec` (:90-205), `GemmMappingSpec`
(:213-446), `OperandLayout` (:454-501), `WeakScaledMappedGemmInstance`
(:509-719) with its exact label round trip, plus the older pure validator
`validate_gemm_config` (mlir_kernels/gemm_config.py:11-71).  Field names,
argument meaning, derived quantities, estimator formulas and error behaviour
are the reference's; what is new is additive and defaults to the reference's
behaviour: operand / output element types and the scale mode on `GemmSpec`
(the reference is f16 x f16 -> f32 only, :115-118).

The problem is always C[M, N] += A[M, K] * B[N, K]: B is stored N x K
row-major, i.e. column-major K x N.
"""

from __future__ import annotations

import dataclasses
import math
import re
from dataclasses import dataclass, field
from enum import Enum
from typing import Optional

from .kittens_helpers import PIPELINE_STRATEGIES
from .layout import Layout


class LoadType(Enum):
    FLAT = "flat"
    BUFFER = "buffer"


class OperandPath(Enum):
    LDS = "lds"              # A and B staged through LDS
    DIRECT_B = "direct_b"    # B pre-shuffled, loaded straight into MFMA operands
    DIRECT_AB = "direct_ab"  # neither operand goes through LDS


class Operand(Enum):
    A = "a"
    B = "b"
    C = "c"


A, B, C = Operand.A, Operand.B, Operand.C

DIM_M, DIM_N, DIM_K = 0, 1, 2

# Default f16 MFMA tile per target (reference :74-82).
_MFMA_SHAPE_FOR_MCPU = {"gfx942": [16, 16, 16], "gfx950": [16, 16, 32]}


def mfma_shape_for_mcpu(mcpu: str) -> list:
    return list(_MFMA_SHAPE_FOR_MCPU.get(mcpu, [16, 16, 16]))


# Storage types understood by the HIP kernels: name -> (bytes per element as a
# fraction numerator/denominator).  mxfp4 packs two elements per byte.
DTYPE_BITS = {"f16": 16, "bf16": 16, "fp8_e4m3": 8, "mxfp4": 4, "f32": 32}


class OperandLayout:
    """Geometry of one operand: flat memory layout (byte strides), which GEMM
    dimension each mode is, element width."""

    def __init__(self, memory_layout: Layout, logical_dims: list, elt_bytes: int,
                 mfma_shape: list):
        if not memory_layout.is_flat:
            raise AssertionError(
                f"OperandLayout requires flat memory_layout, got {memory_layout!r}")
        self.memory_layout = memory_layout
        self.logical_dims = logical_dims
        self.elt_bytes = elt_bytes
        self.mfma_shape = mfma_shape

    @staticmethod
    def _as_tuple(v) -> tuple:
        return v if isinstance(v, tuple) else (v,)

    @property
    def rank(self) -> int:
        return len(self.memory_layout)

    @property
    def shape(self) -> tuple:
        return self._as_tuple(self.memory_layout.sizes)

    @property
    def strides(self) -> tuple:
        return self._as_tuple(self.memory_layout.strides)

    @property
    def num_elements(self) -> int:
        return self.memory_layout.size()


def _packed_layout(sizes: tuple, elt_bytes: int) -> Layout:
    strides, pitch = [], elt_bytes
    for sz in reversed(sizes):
        strides.insert(0, pitch)
        pitch *= sz
    return Layout(tuple(sizes), tuple(strides))


@dataclass
class GemmSpec:
    """The GEMM problem: per-operand memory layouts (source of truth for sizes and
    byte strides), logical dims, MFMA tile shape, element widths."""

    layout_a: Layout
    layout_b: Layout
    layout_c: Layout
    logical_dims_a: list = field(default_factory=lambda: [DIM_M, DIM_K])
    logical_dims_b: list = field(default_factory=lambda: [DIM_N, DIM_K])
    logical_dims_c: list = field(default_factory=lambda: [DIM_M, DIM_N])
    mfma_shape: list = field(default_factory=lambda: [16, 16, 16])
    elt_bytes_a: int = 2
    elt_bytes_b: int = 2
    elt_bytes_c: int = 4
    # --- additions of this build (defaults = the reference's only case) ---
    dtype_ab: str = "f16"      # "f16" | "bf16" | "fp8_e4m3" | "mxfp4"
    dtype_c: str = "f32"       # "f32" | "bf16" | "f16"
    scale_mode: str = "none"   # "none" | "tensor" (fp32 per operand) | "mx32" (e8m0 per 32 K)
    has_bias: bool = False

    def __post_init__(self):
        if self.dtype_ab not in ("f16", "bf16", "fp8_e4m3", "mxfp4"):
            raise ValueError(f"unknown dtype_ab {self.dtype_ab!r}")
        if self.dtype_c not in ("f32", "bf16", "f16"):
            raise ValueError(f"unknown dtype_c {self.dtype_c!r}")
        if self.scale_mode not in ("none", "tensor", "mx32"):
            raise ValueError(f"unknown scale_mode {self.scale_mode!r}")
        mk = lambda lay, dims, eb: OperandLayout(lay, dims, eb, self.mfma_shape)
        self._operand_layouts = {
            Operand.A: mk(self.layout_a, self.logical_dims_a, self.elt_bytes_a),
            Operand.B: mk(self.layout_b, self.logical_dims_b, self.elt_bytes_b),
            Operand.C: mk(self.layout_c, self.logical_dims_c, self.elt_bytes_c),
        }

    @classmethod
    def from_sizes(cls, M: int, N: int, K: int, *, elt_bytes_a: int = 2, elt_bytes_b: int = 2,
                   elt_bytes_c: int = 4, logical_dims_a: Optional[list] = None,
                   logical_dims_b: Optional[list] = None, logical_dims_c: Optional[list] = None,
                   **kwargs) -> "GemmSpec":
        """Packed row-major layouts from the problem sizes."""
        extent = {DIM_M: M, DIM_N: N, DIM_K: K}
        dims = [logical_dims_a or [DIM_M, DIM_K], logical_dims_b or [DIM_N, DIM_K],
                logical_dims_c or [DIM_M, DIM_N]]
        widths = [elt_bytes_a, elt_bytes_b, elt_bytes_c]
        lays = [_packed_layout(tuple(extent[d] for d in ds), eb) for ds, eb in zip(dims, widths)]
        return cls(layout_a=lays[0], layout_b=lays[1], layout_c=lays[2],
                   logical_dims_a=dims[0], logical_dims_b=dims[1], logical_dims_c=dims[2],
                   elt_bytes_a=elt_bytes_a, elt_bytes_b=elt_bytes_b, elt_bytes_c=elt_bytes_c,
                   **kwargs)

    @classmethod
    def from_dtypes(cls, M: int, N: int, K: int, dtype_ab: str = "f16", dtype_c: str = "f32",
                    **kwargs) -> "GemmSpec":
        """Like `from_sizes`, element widths derived from the storage types
        (mxfp4 rows are described in whole bytes: elt_bytes 1 with K/2 columns is
        not expressible, so its layout keeps elt_bytes 1 and the kernels take the
        packed row pitch K/2)."""
        eb_ab = max(1, DTYPE_BITS[dtype_ab] // 8)
        scale_mode = kwargs.pop("scale_mode", None)
        if scale_mode is None:
            scale_mode = {"fp8_e4m3": "tensor", "mxfp4": "mx32"}.get(dtype_ab, "none")
        mfma = kwargs.pop("mfma_shape", None)
        if mfma is None:
            mfma = {"fp8_e4m3": [16, 16, 128], "mxfp4": [16, 16, 128]}.get(dtype_ab, [16, 16, 32])
        return cls.from_sizes(M, N, K, elt_bytes_a=eb_ab, elt_bytes_b=eb_ab,
                              elt_bytes_c=DTYPE_BITS[dtype_c] // 8, dtype_ab=dtype_ab,
                              dtype_c=dtype_c, scale_mode=scale_mode, mfma_shape=mfma, **kwargs)

    def operand_layout(self, operand: Operand) -> OperandLayout:
        return self._operand_layouts[operand]

    def _dim_from_operand(self, operand: Operand, dim: int) -> int:
        ol = self.operand_layout(operand)
        return ol.shape[ol.logical_dims.index(dim)]

    @property
    def gemm_size(self) -> list:
        """[M, N, K] read back from the operand layouts."""
        return [self._dim_from_operand(Operand.A, DIM_M), self._dim_from_operand(Operand.B, DIM_N),
                self._dim_from_operand(Operand.A, DIM_K)]

    def operand_shape(self, operand: Operand) -> tuple:
        return self.operand_layout(operand).shape

    @property
    def total_flops(self) -> int:
        m, n, k = self.gemm_size
        return 2 * m * n * k

    @property
    def total_bytes(self) -> int:
        """Algorithmic HBM bytes: A + B (+ e8m0 planes) + C."""
        m, n, k = self.gemm_size
        ab = (m + n) * k * DTYPE_BITS[self.dtype_ab] // 8
        if self.scale_mode == "mx32":
            ab += (m + n) * (k // 32)
        if self.scale_mode == "tensor":
            ab += 8
        return ab + m * n * self.elt_bytes_c + (4 * n if self.has_bias else 0)


@dataclass
class GemmMappingSpec:
    """How the GEMM is laid onto workgroups, waves and MFMA tiles, plus the
    scheduling knobs the reference's compiler consumes.  The hand-written kernels
    read the geometry (workgroup tile, wave grid) to pick a variant; the
    scheduling knobs are kept so that labels round-trip and estimators agree."""

    num_workgroups_per_kernel: list          # [M, N, K]; K is always 1
    num_waves_per_workgroup: list            # [M, N, K]; K is always 1
    num_tiles_per_wave: list                 # [M, N, K] per K-loop iteration
    tile_mult: list = field(default_factory=lambda: [1, 1, 2])
    pipeline_strategy: int = 1
    load_type: LoadType = LoadType.FLAT
    operand_path: OperandPath = OperandPath.LDS
    lcm_unroll: bool = True
    unroll_factor_multiplier: int = 1
    prologue_peeling: int = 0
    epilogue_peeling: bool = True
    ll_sched: int = 0
    hoist_wait: bool = False
    set_mfma_priority: bool = False
    rotate_compute_stage: bool = False
    use_conservative_barriers: bool = False
    global_load_bytes: int = 16
    ds_write_bytes: int = 8
    ds_read_bytes: int = 8
    mcpu: str = "gfx942"
    num_wg_per_cu: int = 1
    wave_size: int = 64

    VGPRS_PER_LOAD = 4          # one dwordx4
    AGPRS_PER_MFMA_RESULT = 4   # one 16x16 f32 fragment

    def _pipeline_stage_dict(self) -> dict:
        return PIPELINE_STRATEGIES[self.pipeline_strategy]

    @property
    def rotate_stage(self) -> Optional[int]:
        return self._pipeline_stage_dict()["COMPUTE"] if self.rotate_compute_stage else None

    @property
    def isa(self) -> str:
        return {"gfx942": "cdna3", "gfx950": "cdna4"}.get(self.mcpu, "cdna3")

    def tile_elements(self, mfma_shape: list) -> list:
        return [s * m for s, m in zip(mfma_shape, self.tile_mult)]

    @staticmethod
    def default_tile_elements(mfma_shape: list, tile_mult: Optional[list] = None) -> list:
        return [s * m for s, m in zip(mfma_shape, tile_mult or [1, 1, 2])]

    @property
    def num_tiles_per_workgroup(self) -> list:
        return [t * w for t, w in zip(self.num_tiles_per_wave, self.num_waves_per_workgroup)]

    @property
    def num_workgroups(self) -> int:
        return math.prod(self.num_workgroups_per_kernel[:3])

    @property
    def num_waves(self) -> int:
        return math.prod(self.num_waves_per_workgroup[:3])

    @property
    def num_threads(self) -> int:
        return self.num_waves * self.wave_size

    @property
    def direct_b(self) -> bool:
        return self.operand_path in (OperandPath.DIRECT_B, OperandPath.DIRECT_AB)

    @property
    def direct_a(self) -> bool:
        return self.operand_path == OperandPath.DIRECT_AB

    @property
    def use_buffer(self) -> bool:
        return self.load_type == LoadType.BUFFER

    # ---- resource estimates (reference :358-446) ----------------------------

    def estimated_agprs(self) -> int:
        return (self.num_tiles_per_wave[DIM_M] * self.num_tiles_per_wave[DIM_N]
                * self.AGPRS_PER_MFMA_RESULT)

    def _operand_vgprs(self, s: dict, prefix: str, coop_tiles: int) -> int:
        """Steady-state VGPRs of one pipelined operand: buffers live between the
        producing and consuming stage, per tile (reference :365-386)."""
        mt, nt, kt = self.num_tiles_per_wave
        tiles = mt * kt if prefix == "A" else kt * nt
        load, compute = s[f"{prefix}_LOAD"], s["COMPUTE"]
        if (prefix == "B" and self.direct_b) or (prefix == "A" and self.direct_a):
            return tiles * (compute - load + 1) * self.VGPRS_PER_LOAD
        deep = max(0, compute - 2)
        in_flight = coop_tiles * (s[f"{prefix}_LDS_WRITE"] - load + 1)
        fragments = tiles * (compute - s[f"{prefix}_LDS_READ"] + 1 + deep)
        return (in_flight + fragments) * self.VGPRS_PER_LOAD

    def _coop_tiles_per_wave(self) -> tuple:
        kt, nw = self.num_tiles_per_wave[DIM_K], self.num_waves
        twg = self.num_tiles_per_workgroup

        def split(num_tiles: int) -> int:
            ws = min(num_tiles, nw)
            wk = max(1, nw // ws)
            return math.ceil(num_tiles / ws) * math.ceil(kt / wk)

        return split(twg[DIM_M]), split(twg[DIM_N])

    def estimated_vgprs(self) -> int:
        s = self._pipeline_stage_dict()
        coop_a, coop_b = self._coop_tiles_per_wave()
        return self._operand_vgprs(s, "A", coop_a) + self._operand_vgprs(s, "B", coop_b) + 10

    def lds_bytes(self, tile_bytes: int = 1024, **overrides) -> int:
        """LDS live between allocation (earliest load stage) and the LDS-read
        stage, multi-buffered by that stage distance (reference :414-441)."""
        kt = self.num_tiles_per_wave[DIM_K]
        s = self._pipeline_stage_dict()
        alloc = s["A_LOAD"] if self.direct_b else min(s["A_LOAD"], s["B_LOAD"])
        twg = self.num_tiles_per_workgroup
        total = max(1, s["A_LDS_READ"] - alloc + 1) * twg[DIM_M] * kt * tile_bytes
        if not self.direct_b:
            total += max(1, s["B_LDS_READ"] - alloc + 1) * kt * twg[DIM_N] * tile_bytes
        return total

    def simd_occupancy(self) -> int:
        return self.num_wg_per_cu * math.ceil(self.num_waves / 4)


_LABEL_RE = re.compile(
    r"^m(\d+)xn(\d+)xk(\d+)"
    r"_wg(\d+)x(\d+)x(\d+)_w(\d+)x(\d+)x(\d+)"
    r"_twg(\d+)x(\d+)x(\d+)_pipestrat(\d+)"
    r"_wgcu(\d+)_lcm([01])_um(\d+)_epeel([01])_llsched(\d+)_hoistwait([01])_rotc([01])"
    r"(?:_consbar([01]))?"
    r"_lt_(flat|buf)$"
)


class WeakScaledMappedGemmInstance:
    """A GemmSpec + GemmMappingSpec pair whose sizes satisfy the weak-scale rule
    M == workgroups[M] * tiles_per_workgroup[M] * mfma_m (same for N); unknown
    attributes are looked up on the spec, then on the mapping."""

    _KERNEL_NAMES = {
        OperandPath.LDS: "gemm_f16_weak_scaled",
        OperandPath.DIRECT_B: "gemm_f16_direct_b",
        OperandPath.DIRECT_AB: "gemm_f16_direct_ab",
    }

    def __init__(self, spec: GemmSpec, mapping: GemmMappingSpec):
        self.spec = spec
        self.mapping = mapping
        self._check_weak_scale()

    def _check_weak_scale(self) -> None:
        wg, twg = self.mapping.num_workgroups_per_kernel, self.mapping.num_tiles_per_workgroup
        gs, mfma = self.spec.gemm_size, self.spec.mfma_shape
        for dim, name in ((DIM_M, "M"), (DIM_N, "N")):
            want = wg[dim] * twg[dim] * mfma[dim]
            assert gs[dim] == want, (
                f"gemm_size[{name}]={gs[dim]} != num_workgroups_per_kernel[{name}]({wg[dim]}) * "
                f"num_tiles_per_wg[{name}]({twg[dim]}) * mfma_shape[{name}]({mfma[dim]}) = {want}")

    @property
    def gemm_size(self) -> list:
        return self.spec.gemm_size

    @property
    def load_type(self) -> str:
        return self.mapping.load_type.value

    @property
    def b_path(self) -> str:
        return self.mapping.operand_path.value

    @property
    def estimated_agprs(self) -> int:
        return self.mapping.estimated_agprs()

    @property
    def estimated_vgprs(self) -> int:
        return self.mapping.estimated_vgprs()

    @property
    def lds_bytes(self) -> int:
        return self.mapping.lds_bytes()

    @property
    def simd_occupancy(self) -> int:
        return self.mapping.simd_occupancy()

    @property
    def kernel_name(self) -> str:
        return self._KERNEL_NAMES[self.mapping.operand_path]

    @property
    def k_scaling_factor(self) -> int:
        tile_k = self.mapping.tile_elements(self.spec.mfma_shape)[DIM_K]
        return self.gemm_size[DIM_K] // (self.mapping.num_tiles_per_wave[DIM_K] * tile_k)

    # ---- label serde: every knob is always written, round trip is exact ----

    @property
    def label(self) -> str:
        m = self.mapping
        gs = self.gemm_size
        x3 = lambda v: "x".join(str(i) for i in v[:3])
        parts = [
            f"m{gs[DIM_M]}xn{gs[DIM_N]}xk{gs[DIM_K]}",
            f"wg{x3(m.num_workgroups_per_kernel)}",
            f"w{x3(m.num_waves_per_workgroup)}",
            f"twg{x3(self.num_tiles_per_workgroup)}",
            f"pipestrat{m.pipeline_strategy}",
            f"wgcu{m.num_wg_per_cu}",
            f"lcm{int(m.lcm_unroll)}",
            f"um{m.unroll_factor_multiplier}",
            f"epeel{int(m.epilogue_peeling)}",
            f"llsched{int(m.ll_sched)}",
            f"hoistwait{int(m.hoist_wait)}",
            f"rotc{int(m.rotate_compute_stage)}",
            f"consbar{int(m.use_conservative_barriers)}",
            "lt_" + ("buf" if m.load_type == LoadType.BUFFER else "flat"),
        ]
        return "_".join(parts)

    @staticmethod
    def canonical_label(label: str) -> str:
        """Labels written before the barrier knob existed lack `_consbarN`; the
        canonical form spells it out."""
        if "_consbar" in label:
            return label
        return re.sub(r"_lt_(flat|buf)", r"_consbar0_lt_\1", label, count=1)

    @classmethod
    def _parse_label(cls, label: str):
        mt = _LABEL_RE.match(label)
        if not mt:
            raise ValueError(f"Cannot parse label: {label}")
        g = mt.groups()
        nums = [int(v) for v in g[:13]]
        M, N, K = nums[0:3]
        wg, wpw, twg = nums[3:6], nums[6:9], nums[9:12]
        if any(w == 0 for w in wpw):
            raise ValueError(f"Cannot parse label: {label} (zero waves)")
        spec = GemmSpec.from_sizes(M, N, K)
        mapping = GemmMappingSpec(
            num_workgroups_per_kernel=wg,
            num_waves_per_workgroup=wpw,
            num_tiles_per_wave=[t // w for t, w in zip(twg, wpw)],
            pipeline_strategy=nums[12],
            load_type=LoadType.BUFFER if g[21] == "buf" else LoadType.FLAT,
            num_wg_per_cu=int(g[13]),
            lcm_unroll=g[14] == "1",
            unroll_factor_multiplier=int(g[15]),
            epilogue_peeling=g[16] == "1",
            ll_sched=int(g[17]),
            hoist_wait=g[18] == "1",
            rotate_compute_stage=g[19] == "1",
            use_conservative_barriers=(g[20] == "1") if g[20] is not None else False,
        )
        return spec, mapping

    @classmethod
    def from_label(cls, label: str) -> "WeakScaledMappedGemmInstance":
        spec, mapping = cls._parse_label(label)
        cfg = cls(spec, mapping)
        want = cls.canonical_label(label)
        assert cfg.label == want, f"Round-trip failed: {cfg.label!r} != {want!r}"
        return cfg

    def __getattr__(self, name: str):
        if name in ("spec", "mapping"):  # not yet set (e.g. while unpickling)
            raise AttributeError(name)
        for holder in ("spec", "mapping"):
            try:
                return getattr(object.__getattribute__(self, holder), name)
            except AttributeError:
                continue
        raise AttributeError(f"'{type(self).__name__}' has no attribute '{name}'") from None


class Cdna4GemmInstance(WeakScaledMappedGemmInstance):
    """gfx950 instance: 16x16x32 MFMA, label suffix `_cdna4`
    (reference: contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:328-383)."""

    KERNEL_NAME = "gemm_cdna4"

    @property
    def kernel_name(self) -> str:
        return self.KERNEL_NAME

    @property
    def transfer_tile_k_elems(self) -> int:
        return self.spec.mfma_shape[DIM_K]

    @property
    def transfer_tile_row_bytes(self) -> int:
        return self.transfer_tile_k_elems * self.spec.elt_bytes_a

    @property
    def transfer_tile_bytes(self) -> int:
        return self.spec.mfma_shape[DIM_M] * self.transfer_tile_row_bytes

    @property
    def label(self) -> str:
        return f"{super().label}_cdna4"

    @classmethod
    def from_label(cls, label: str, operand_path: OperandPath = OperandPath.DIRECT_B
                   ) -> "Cdna4GemmInstance":
        core = label[: -len("_cdna4")] if label.endswith("_cdna4") else label
        spec, mapping = cls._parse_label(core)
        spec = GemmSpec.from_sizes(*spec.gemm_size, mfma_shape=mfma_shape_for_mcpu("gfx950"))
        mapping = dataclasses.replace(mapping, operand_path=operand_path,
                                      load_type=LoadType.FLAT, mcpu="gfx950")
        cfg = cls(spec, mapping)
        want = cls.canonical_label(core) + "_cdna4"
        assert cfg.label == want, f"Round-trip failed: {cfg.label!r} != {want!r}"
        return cfg


def make_instance(M: int, N: int, K: int, *, dtype_ab: str = "bf16", dtype_c: str = "bf16",
                  wg_tile=(256, 256), waves=(2, 4), pipeline_strategy: int = 1,
                  has_bias: bool = False, scale_mode: Optional[str] = None,
                  operand_path: "OperandPath" = None) -> WeakScaledMappedGemmInstance:
    """Instance for one of the HIP kernels' native tilings: M and N must be
    multiples of the workgroup tile (the weak-scale rule)."""
    tm, tn = wg_tile
    if M % tm or N % tn:
        raise AssertionError(f"M={M}, N={N} not multiples of the workgroup tile {tm}x{tn}")
    spec = GemmSpec.from_dtypes(M, N, K, dtype_ab, dtype_c, has_bias=has_bias,
                                scale_mode=scale_mode)
    mfma = spec.mfma_shape
    mapping = GemmMappingSpec(
        num_workgroups_per_kernel=[M // tm, N // tn, 1],
        num_waves_per_workgroup=[waves[0], waves[1], 1],
        num_tiles_per_wave=[tm // mfma[0] // waves[0], tn // mfma[1] // waves[1], 1],
        pipeline_strategy=pipeline_strategy,
        mcpu="gfx950",
        **({} if operand_path is None else {"operand_path": operand_path}),
    )
    return WeakScaledMappedGemmInstance(spec, mapping)


def is_power_of_two(n: int) -> bool:
    return n > 0 and n & (n - 1) == 0


def validate_gemm_config(m: int, n: int, k: int, m_tile: int, n_tile: int, k_tile: int,
                         num_waves: int = 1):
    """(ok, reason) for the older dword4 16x16x16 tiling rules
    (reference: mlir_kernels/gemm_config.py:11-71); reasons are the reference's."""
    dims = (("M", m, "m_tile", m_tile), ("N", n, "n_tile", n_tile), ("K", k, "k_tile", k_tile))
    for big, size, name, t in dims:
        if size % t != 0:
            return False, f"{big} must be a multiple of {name}"
    for _, _, name, t in dims:
        if t % 16 != 0:
            return False, f"{name} must be a multiple of 16"
    for _, _, name, t in dims:
        if t < 16:
            return False, f"{name} must be at least 16"
    for _, _, name, t in dims:
        if not is_power_of_two(t // 16):
            return False, f"{name} / 16 must be a power of 2"
    if num_waves <= 0:
        return False, "Number of waves must be positive"
    if not is_power_of_two(num_waves):
        return False, "Number of waves must be a power of 2"
    mb, nb, kb = m_tile // 16, n_tile // 16, k_tile // 16
    for prod, text in ((mb * nb, "m_tile/16 * n_tile/16"), (mb * kb, "m_tile/16 * k_tile/16"),
                       (kb * nb, "k_tile/16 * n_tile/16")):
        if prod % num_waves != 0:
            return False, f"{text} must be divisible by num_waves"
    return True, None
