"""Config surface: label round trips on the reference's own cases, estimator
anchors, validators."""
import json
import os

import pytest

from aster_amd.gemm_config import (DIM_K, DIM_M, DIM_N, Cdna4GemmInstance, GemmMappingSpec, GemmSpec,
                                   LoadType, OperandPath, WeakScaledMappedGemmInstance, make_instance,
                                   mfma_shape_for_mcpu, validate_gemm_config)
from aster_amd.kittens_helpers import PIPELINE_STRATEGIES, pipeline_strategy_stages
from aster_amd.layout import Layout


def _make(num_workgroups_per_kernel, num_waves_per_wg, num_tiles_per_wg, k, pipeline_strategy=1,
          load_type="flat", b_path="lds", **kw):
    """Same construction as the reference's test helper
    (contrib/kittens/test/test_perf_001_gemm_fp16_weak_scaled.py:60-95)."""
    twg, wpw = num_tiles_per_wg, num_waves_per_wg
    M = num_workgroups_per_kernel[0] * twg[0] * 16
    N = num_workgroups_per_kernel[1] * twg[1] * 16
    spec = GemmSpec.from_sizes(M, N, k)
    mapping = GemmMappingSpec(
        num_workgroups_per_kernel=list(num_workgroups_per_kernel),
        num_waves_per_workgroup=list(wpw),
        num_tiles_per_wave=[twg[0] // wpw[0], twg[1] // wpw[1], twg[2] // wpw[2]],
        pipeline_strategy=pipeline_strategy, load_type=LoadType(load_type),
        operand_path=OperandPath(b_path), **kw)
    return WeakScaledMappedGemmInstance(spec, mapping)


# The 18 parametrisations of TestWeakScaledMappedGemmInstanceSerde
# (test_perf_001_gemm_fp16_weak_scaled.py:365-450).
SERDE_CASES = [
    dict(), dict(load_type="buffer"), dict(b_path="direct_b"),
    dict(load_type="buffer", b_path="direct_b"), dict(b_path="direct_ab"),
    dict(load_type="buffer", b_path="direct_ab"),
    dict(num_wg_per_cu=2, num_workgroups_per_kernel=[38, 16, 1]),
    dict(num_wg_per_cu=4, num_workgroups_per_kernel=[76, 16, 1]),
    dict(lcm_unroll=False), dict(unroll_factor_multiplier=3), dict(epilogue_peeling=False),
    dict(ll_sched=True), dict(hoist_wait=True), dict(rotate_compute_stage=False),
    dict(pipeline_strategy=0), dict(pipeline_strategy=5), dict(pipeline_strategy=9),
    dict(lcm_unroll=False, unroll_factor_multiplier=2, epilogue_peeling=False, ll_sched=True,
         hoist_wait=True, rotate_compute_stage=False, num_wg_per_cu=2,
         num_workgroups_per_kernel=[38, 16, 1], load_type="buffer", b_path="direct_b",
         pipeline_strategy=7),
]


@pytest.mark.parametrize("kwargs", SERDE_CASES)
def test_label_roundtrip(kwargs):
    base = dict(num_workgroups_per_kernel=[19, 16, 1], num_waves_per_wg=[2, 2, 1],
                num_tiles_per_wg=[8, 8, 2], k=8192, pipeline_strategy=1)
    base.update(kwargs)
    cfg = _make(**base)
    restored = WeakScaledMappedGemmInstance.from_label(cfg.label)
    assert restored.label == cfg.label
    for f in ["gemm_size", "pipeline_strategy", "load_type", "num_wg_per_cu", "lcm_unroll",
              "unroll_factor_multiplier", "epilogue_peeling", "ll_sched", "hoist_wait",
              "rotate_compute_stage", "use_conservative_barriers", "num_workgroups_per_kernel",
              "num_waves_per_workgroup", "num_tiles_per_workgroup", "num_threads"]:
        assert getattr(restored, f) == getattr(cfg, f), f


def test_default_label_text():
    cfg = _make([19, 16, 1], [2, 2, 1], [8, 8, 2], k=8192)
    assert cfg.label == ("m2432xn2048xk8192_wg19x16x1_w2x2x1_twg8x8x2_pipestrat1_wgcu1_lcm1_um1_"
                         "epeel1_llsched0_hoistwait0_rotc0_consbar0_lt_flat")


def test_from_label_rejects_garbage_and_truncated():
    with pytest.raises(ValueError, match="Cannot parse label"):
        WeakScaledMappedGemmInstance.from_label("not_a_valid_label")
    cfg = _make([19, 16, 1], [2, 2, 1], [8, 8, 1], k=4096)
    with pytest.raises(ValueError):
        WeakScaledMappedGemmInstance.from_label(cfg.label[:-5])


def test_registry_labels_roundtrip(golden_dir):
    with open(os.path.join(golden_dir, "best_known_labels.json")) as f:
        entries = json.load(f)
    assert len(entries) == 19
    for e in entries:
        lab = e["label"]
        if lab.endswith("_cdna4"):
            cfg = Cdna4GemmInstance.from_label(lab)
            assert cfg.spec.mfma_shape == [16, 16, 32] and cfg.mapping.direct_b
            assert cfg.label == WeakScaledMappedGemmInstance.canonical_label(lab[:-6]) + "_cdna4"
        else:
            cfg = WeakScaledMappedGemmInstance.from_label(lab)
            assert cfg.label == WeakScaledMappedGemmInstance.canonical_label(lab)
        m, n, k = (int(v) for v in e["size"].split("x"))
        assert cfg.gemm_size == [m, n, k]
        assert cfg.total_flops == 2 * m * n * k


def test_best_gfx950_mapping_geometry(golden_dir):
    with open(os.path.join(golden_dir, "best_known_labels.json")) as f:
        best = max((e for e in json.load(f) if e["mcpu"] == "gfx950"), key=lambda e: e["expected_tflops"])
    assert best["expected_tflops"] == 1007.0
    cfg = Cdna4GemmInstance.from_label(best["label"])
    twg = cfg.num_tiles_per_workgroup
    assert [twg[0] * 16, twg[1] * 16] == [128, 256] and cfg.num_threads == 256
    assert cfg.mapping.num_workgroups == 512


def test_estimator_anchors(golden_dir):
    with open(os.path.join(golden_dir, "kat.json")) as f:
        anchors = json.load(f)["estimator_anchors"]
    for a in anchors:
        cfg = Cdna4GemmInstance.from_label(a["label"], OperandPath(a["operand_path"]))
        assert cfg.estimated_vgprs == a["vgprs"]
        assert cfg.estimated_agprs == a["agprs"]
        assert cfg.lds_bytes == a["lds"]
        if "simd_occupancy" in a:
            assert cfg.simd_occupancy == a["simd_occupancy"]
    lds = _make([1, 1, 1], [2, 2, 1], [4, 4, 1], k=256, pipeline_strategy=3)
    assert (lds.estimated_vgprs, lds.estimated_agprs, lds.lds_bytes) == (42, 16, 24576)


def test_gemm_spec_layouts_and_sizes():
    s = GemmSpec.from_sizes(64, 48, 32)
    assert s.gemm_size == [64, 48, 32] and s.total_flops == 2 * 64 * 48 * 32
    assert s.layout_a == Layout((64, 32), (64, 2))       # byte strides, f16
    assert s.layout_b == Layout((48, 32), (64, 2))       # B stored N x K
    assert s.layout_c == Layout((64, 48), (192, 4))      # f32
    assert s.operand_shape(__import__("aster_amd").B) == (48, 32)
    assert (s.elt_bytes_a, s.elt_bytes_b, s.elt_bytes_c) == (2, 2, 4)
    assert mfma_shape_for_mcpu("gfx950") == [16, 16, 32] and mfma_shape_for_mcpu("gfx942") == [16, 16, 16]
    assert mfma_shape_for_mcpu("other") == [16, 16, 16]


def test_weak_scale_rule_is_enforced():
    spec = GemmSpec.from_sizes(100, 64, 64)
    mapping = GemmMappingSpec([1, 1, 1], [2, 2, 1], [2, 2, 1])
    with pytest.raises(AssertionError, match="gemm_size"):
        WeakScaledMappedGemmInstance(spec, mapping)


def test_mapping_derived_quantities():
    m = GemmMappingSpec([32, 16, 1], [1, 4, 1], [8, 4, 1], mcpu="gfx950",
                        operand_path=OperandPath.DIRECT_B)
    assert m.num_tiles_per_workgroup == [8, 16, 1]
    assert (m.num_workgroups, m.num_waves, m.num_threads) == (512, 4, 256)
    assert m.direct_b and not m.direct_a and not m.use_buffer and m.isa == "cdna4"
    assert m.tile_elements([16, 16, 32]) == [16, 16, 64]
    assert m.rotate_stage is None
    cfg = WeakScaledMappedGemmInstance(GemmSpec.from_sizes(4096, 4096, 4096), m)
    assert cfg.kernel_name == "gemm_f16_direct_b" and cfg.b_path == "direct_b"
    assert cfg.k_scaling_factor == 4096 // 32
    with pytest.raises(AttributeError):
        cfg.no_such_field


def test_pipeline_strategies_table():
    assert len(PIPELINE_STRATEGIES) == 14
    for i in range(11):  # shared barrier invariant of strategies 0-10
        assert PIPELINE_STRATEGIES[i]["A_LDS_READ"] == PIPELINE_STRATEGIES[i]["B_LDS_READ"]
    assert PIPELINE_STRATEGIES[11] == dict(A_LOAD=0, A_LDS_WRITE=1, A_LDS_READ=3, B_LOAD=0,
                                           B_LDS_WRITE=1, B_LDS_READ=4, COMPUTE=4)
    assert pipeline_strategy_stages(0) == (1, 1)
    assert pipeline_strategy_stages(11) == (5, 5)
    assert pipeline_strategy_stages(5) == (4, 4)


def test_dtype_extension_defaults_keep_reference_behaviour():
    s = GemmSpec.from_sizes(16, 16, 32)
    assert (s.dtype_ab, s.dtype_c, s.scale_mode, s.has_bias) == ("f16", "f32", "none", False)
    b = GemmSpec.from_dtypes(8192, 8192, 8192, "bf16", "bf16")
    assert b.total_bytes == 402653184                 # config 2 of the baseline
    f = GemmSpec.from_dtypes(8192, 8192, 8192, "fp8_e4m3", "bf16")
    assert f.scale_mode == "tensor" and f.total_bytes == 268435464
    x = GemmSpec.from_dtypes(4096, 14336, 4096, "mxfp4", "bf16")
    assert x.scale_mode == "mx32" and x.total_bytes == 157548544
    d = GemmSpec.from_dtypes(16, 14336, 4096, "bf16", "bf16")
    assert d.total_bytes == 118030336
    with pytest.raises(ValueError):
        GemmSpec.from_sizes(16, 16, 32, dtype_ab="int8")
    inst = make_instance(8192, 8192, 8192)
    assert inst.num_workgroups == 1024 and inst.num_threads == 512
    with pytest.raises(AssertionError):
        make_instance(100, 256, 64)


@pytest.mark.parametrize("args,ok,reason", [
    ((256, 256, 256, 64, 64, 32, 4), True, None),
    ((250, 256, 256, 64, 64, 32, 4), False, "M must be a multiple of m_tile"),
    ((256, 256, 250, 64, 64, 32, 4), False, "K must be a multiple of k_tile"),
    ((240, 240, 240, 24, 16, 16, 1), False, "m_tile must be a multiple of 16"),
    ((96, 96, 96, 48, 16, 16, 1), False, "m_tile / 16 must be a power of 2"),
    ((256, 256, 256, 64, 64, 32, 0), False, "Number of waves must be positive"),
    ((256, 256, 256, 64, 64, 32, 3), False, "Number of waves must be a power of 2"),
    ((256, 256, 256, 16, 16, 16, 2), False, "m_tile/16 * n_tile/16 must be divisible by num_waves"),
    ((256, 256, 256, 32, 16, 16, 2), False, "k_tile/16 * n_tile/16 must be divisible by num_waves"),
])
def test_validate_gemm_config(args, ok, reason):
    assert validate_gemm_config(*args) == (ok, reason)
