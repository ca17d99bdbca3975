"""Host-side contracts that need no GPU: C-ABI exports, config validation and
variant selection, kernel-argument packing, array roles, bench statistics."""
import ctypes
import io
import json
import os
import re

import numpy as np
import pytest

from aster_amd import _capi, bench_harness as BH, gemm, make_instance
from aster_amd.execution import (InOutArray, InputArray, OutputArray, create_kernel_args,
                                 create_kernel_args_capsule)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    text = open(os.path.join(ROOT, "include", "astergemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(astergemm_[a-z0-9_]+|aster_rt_[a-z0-9_]+)\s*\(", text))
    assert len(declared) >= 35
    lib = _capi.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in astergemm.h but not exported"
    assert declared == set(_capi.SIGNATURES), declared ^ set(_capi.SIGNATURES)
    assert lib.astergemm_abi_version() == _capi.ABI_VERSION


def test_struct_sizes_match_header_layout():
    # 6 x int64 + 16 x int32 ; pointers ; see include/astergemm.h
    assert ctypes.sizeof(_capi.Config) == 6 * 8 + 16 * 4
    assert ctypes.sizeof(_capi.Operands) == 10 * 8
    assert ctypes.sizeof(_capi.KernelInfo) == 13 * 4 + 4 + 2 * 8 + 64


def test_select_headline_configs():
    p = gemm.GemmPlan.create(8192, 8192, 8192, "bf16", "bf16")
    assert p.info.family == _capi.KERNEL_TILE
    assert p.info.flops == 2 * 8192 ** 3 and p.info.bytes == 402653184
    assert p.info.grid_x * p.info.wg_tile_m * p.info.wg_tile_n == 8192 * 8192
    p = gemm.GemmPlan.create(8192, 8192, 8192, "fp8_e4m3", "bf16")
    assert p.info.bytes == 268435464 and p.info.wg_tile_k == 128
    assert gemm.GemmPlan.create(3072, 3072, 3072, "fp8_e4m3", "bf16").info.name.decode().startswith("stream_fp8_256")
    assert gemm.GemmPlan.create(2048, 4096, 4096, "fp8_e4m3", "bf16").info.name.decode().startswith("stream_fp8_128")
    assert gemm.GemmPlan.create(3072, 3072, 3072, "mxfp4", "bf16").info.name.decode().startswith("stream_mxfp4_128")
    assert gemm.GemmPlan.create(4096, 14336, 4096, "mxfp4", "bf16").info.name.decode().startswith("stream_mxfp4_256")
    assert gemm.GemmPlan.create(96, 4096, 4096, "mxfp4", "bf16").info.name.decode().startswith("stream_mxfp4_128")
    assert gemm.GemmPlan.create(2048, 4096, 4096, "mxfp4", "bf16").info.name.decode().startswith("stream_mxfp4_128")
    # short rows of MXFP4: the tile walk from about two tiles of K = 2048 per CU on, else 128 x 128
    assert gemm.GemmPlan.create(8192, 8192, 1024, "mxfp4", "bf16").info.name.decode() == "stream_mxfp4_256x256_w2x4_walk_bf16"
    assert gemm.GemmPlan.create(4096, 8192, 2048, "mxfp4", "bf16").info.name.decode() == "stream_mxfp4_256x256_w2x4_walk_bf16"
    assert gemm.GemmPlan.create(4096, 8192, 1024, "mxfp4", "bf16").info.name.decode().startswith("stream_mxfp4_128")
    assert gemm.GemmPlan.create(8192, 8192, 512, "mxfp4", "bf16").info.name.decode().startswith("stream_mxfp4_128")
    p = gemm.GemmPlan.create(4096, 14336, 4096, "mxfp4", "bf16")
    assert p.info.bytes == 157548544 and p.info.wg_tile_k == 256
    for M, want in ((1, 117477376), (16, 118030336), (64, 119799808)):
        p = gemm.GemmPlan.create(M, 14336, 4096, "bf16", "bf16")
        assert p.info.family == _capi.KERNEL_SKINNY and p.info.bytes == want
    # tile choice: 256 x 256 once it nearly fills the 256 CUs, else the 128 x 128 stream kernel
    # from 200 workgroups on, else the largest tile with about two workgroups per CU, else the
    # smallest tile
    for (M, N, K), want, kind in (((256, 256, 256), (64, 64), "tile"),
                                  ((2048, 2048, 2048), (128, 128), "stream"),
                                  ((8192, 1024, 8192), (128, 128), "stream"),
                                  ((4096, 4096, 4096), (256, 256), "stream"),
                                  ((128, 14336, 4096), (128, 128), "splitk"),  # 112 tiles, 64 steps
                                  ((128, 4096, 14336), (128, 128), "splitk"),
                                  ((128, 4096, 14344), (64, 64), "tile"),      # K tail: no split
                                  ((640, 4096, 4096), (128, 128), "stream"),   # 160 tiles: no split
                                  ((3000, 5000, 7008), (256, 256), "stream"),
                                  ((2044, 2044, 2048), (128, 64), "tile"),    # M, N not multiples of 8
                                  ((3072, 3072, 3072), (256, 256), "stream"),  # 576 = 512 + 64 tiles of 128
                                  ((2048, 4096, 4096), (128, 128), "stream"),
                                  ((1536, 1536, 8192), (128, 128), "stream")):  # long rows
        p = gemm.GemmPlan.create(M, N, K, "f16", "f32")
        assert p.info.family == _capi.KERNEL_TILE
        assert (p.info.wg_tile_m, p.info.wg_tile_n) == want, (M, N, K)
        assert p.info.name.decode().startswith(kind), (M, N, K)
    # split K: the grid is one copy of the 32 tiles per K range (224 steps in 8 ranges of 28)
    assert gemm.GemmPlan.create(128, 4096, 14336, "bf16", "bf16").info.grid_x == 32 * 8
    assert gemm.GemmPlan.create(128, 4096, 14336, "mxfp4", "bf16").info.grid_x == 32 * 7


def test_explicit_variant_and_enumeration():
    lib = _capi.load()
    n = lib.astergemm_variant_count()
    assert n >= 24
    c = _capi.Config()
    c.M = c.N = c.K = 1024
    c.dtype_ab, c.dtype_c = _capi.BF16, _capi.BF16
    names = set()
    for i in range(n):
        info = _capi.KernelInfo()
        _capi.check(lib.astergemm_variant_info(i, ctypes.byref(c), ctypes.byref(info)))
        assert info.variant == i + 1
        names.add(info.name.decode())
    assert len(names) == n
    info = _capi.KernelInfo()
    assert lib.astergemm_variant_info(n, ctypes.byref(c), ctypes.byref(info)) == -22


@pytest.mark.parametrize("kw,msg", [
    (dict(M=128, N=128, K=0), "K > 0"),
    (dict(M=-1, N=128, K=64), ">= 0"),
    (dict(M=128, N=128, K=100), "16 bytes"),
    (dict(M=128, N=128, K=64, lda=32), "leading dimension"),
    (dict(M=128, N=128, K=64, dtype_ab="mxfp4", dtype_c="bf16", scale_mode="none"), "go together"),
    (dict(M=128, N=128, K=128, dtype_ab="mxfp4", dtype_c="bf16"), "K % 256"),
    (dict(M=128, N=128, K=64, family=_capi.KERNEL_SKINNY), "M <= 64"),
    (dict(M=16, N=128, K=64, dtype_ab="fp8_e4m3", family=_capi.KERNEL_SKINNY), "for fp8"),
    (dict(M=16, N=128, K=1024, dtype_ab="mxfp4", family=_capi.KERNEL_SKINNY), "MXFP4 path"),
])
def test_invalid_configs_are_refused_with_a_reason(kw, msg):
    kw = dict(kw)
    M, N, K = kw.pop("M"), kw.pop("N"), kw.pop("K")
    with pytest.raises(_capi.AsterGemmError) as e:
        gemm.GemmPlan.create(M, N, K, kw.pop("dtype_ab", "bf16"), kw.pop("dtype_c", "bf16"), **kw)
    assert msg in str(e.value)
    assert e.value.code in (-22, -95)


def test_run_refuses_null_and_misaligned_pointers_before_touching_the_gpu():
    p = gemm.GemmPlan.create(256, 256, 256)
    with pytest.raises(_capi.AsterGemmError, match="non-null"):
        p.run(None, None, None)
    with pytest.raises(_capi.AsterGemmError, match="16-byte aligned"):
        p.run(4096 + 8, 4096, 4096)
    q = gemm.GemmPlan.create(256, 256, 256, "fp8_e4m3", "bf16")
    with pytest.raises(_capi.AsterGemmError, match="dScaleA"):
        q.run(4096, 4096, 4096)
    b = gemm.GemmPlan.create(256, 256, 256, has_bias=True)
    with pytest.raises(_capi.AsterGemmError, match="dBias"):
        b.run(4096, 4096, 4096)
    # empty problems are a no-op
    gemm.GemmPlan.create(0, 256, 256).run(4096, 4096, 4096)


def test_compile_gemm_writes_descriptor(tmp_path):
    cfg = make_instance(512, 512, 256)
    path, asm = gemm.compile_gemm(cfg, str(tmp_path / "k.hsaco"), num_vgprs=256, num_agprs=256)
    desc = json.load(open(path))
    assert desc["kernel"] == "stream_bf16_256x256_w2x4_bf16" and desc["grid"] == 4
    assert desc["label"] == cfg.label and desc["lds_bytes"] == 163840
    assert ".group_segment_fixed_size: 163840" in asm
    (tmp_path / "bad.hsaco").write_text("{}")
    with pytest.raises(ValueError):
        gemm._read_descriptor(str(tmp_path / "bad.hsaco"))


def test_descriptor_says_when_the_mapping_is_not_honoured(tmp_path):
    import dataclasses

    from aster_amd.gemm_config import OperandPath, WeakScaledMappedGemmInstance

    # the library's own 256 x 256, 2 x 4 waves geometry: honoured
    cfg = make_instance(512, 512, 256)
    path, asm = gemm.compile_gemm(cfg, str(tmp_path / "a.hsaco"))
    desc = json.load(open(path))
    assert desc["mapping_honoured"] is True and desc["mapping_not_honoured"] == {}
    assert "mapping_honoured: true" in asm
    assert desc["mapping_fixed_by_kernel"]["pipeline_strategy"] == 1
    # the reference's best label geometry (128 x 256 tile, 1 x 4 waves) has no pre-built kernel:
    # the library's choice runs and the descriptor says which requested values it does not have
    cfg = make_instance(512, 512, 256, wg_tile=(128, 256), waves=(1, 4), pipeline_strategy=11)
    path, asm = gemm.compile_gemm(cfg, str(tmp_path / "b.hsaco"))
    desc = json.load(open(path))
    assert desc["mapping_honoured"] is False
    assert desc["mapping_not_honoured"]["wg_tile"]["requested"] == [128, 256]
    assert desc["mapping_not_honoured"]["waves"] == {"requested": [1, 4], "kernel": desc["waves"]}
    assert "mapping_honoured: false" in asm and "wg_tile: requested [128, 256]" in asm
    # a direct_b request on a shape no pre-shuffled kernel takes falls back to row-major B
    m = dataclasses.replace(make_instance(512, 520 // 8 * 8 + 248, 264).mapping,
                            operand_path=OperandPath.DIRECT_B)
    cfg = WeakScaledMappedGemmInstance(make_instance(512, 768, 264).spec, m)
    c, info = gemm.select_for_instance(cfg)
    rep = gemm.mapping_report(cfg, c, info)
    if c.operand_path == _capi.OPERAND_LDS:
        assert rep.not_honoured["operand_path"] == {"requested": "direct_b", "kernel": "lds"}
    else:
        assert "operand_path" not in rep.not_honoured


def test_direct_b_mapping_selects_a_stream_kernel_for_every_operand_type():
    # the reference's best mapping (128 x 256 tile, 1 x 4 waves, B pre-shuffled and loaded straight
    # into MFMA operands) on a compute-bound shape: a kernel of that geometry exists for 16-bit,
    # fp8 and MXFP4 operands, and nothing of the request is reported as dropped
    from aster_amd.gemm_config import OperandPath
    for dt, kernel in (("bf16", "streamdb_bf16_128x256_w1x4"), ("f16", "streamdb_f16_128x256_w1x4"),
                       ("fp8_e4m3", "streamdb_fp8_128x256_w1x4"), ("mxfp4", "streamdb_mxfp4_128x256_w1x4")):
        cfg = make_instance(512, 768, 1024, dtype_ab=dt, wg_tile=(128, 256), waves=(1, 4),
                            operand_path=OperandPath.DIRECT_B)
        c, info = gemm.select_for_instance(cfg)
        assert info.name.decode().startswith(kernel), (dt, info.name)
        assert c.operand_path == _capi.OPERAND_DIRECT_B_K8
        rep = gemm.mapping_report(cfg, c, info)
        assert rep.honoured and not rep.not_honoured, (dt, rep.not_honoured)


def test_direct_ab_mapping_selects_the_kernel_without_lds():
    # reference: operand_path = direct_ab (contrib/kittens/gemm_config.py:213-276) -- A and B both
    # pre-shuffled; here a 16-bit kernel of the 128 x 256, 1 x 4 geometry with no LDS at all
    from aster_amd.gemm_config import OperandPath
    for dt in ("bf16", "f16"):
        cfg = make_instance(512, 768, 640, dtype_ab=dt, wg_tile=(128, 256), waves=(1, 4),
                            operand_path=OperandPath.DIRECT_AB)
        c, info = gemm.select_for_instance(cfg)
        assert info.name.decode().startswith(f"directab_{dt}_128x256_w1x4_"), info.name
        assert c.operand_path == _capi.OPERAND_DIRECT_AB and info.lds_bytes == 0
        assert info.grid_x == 4 * 3 and info.block_x == 256
        rep = gemm.mapping_report(cfg, c, info)
        assert rep.honoured and not rep.not_honoured
    # a row length that does not fill 32-element chunks falls back to the LDS kernels, and says so
    cfg = make_instance(512, 768, 264, operand_path=OperandPath.DIRECT_AB)
    c, info = gemm.select_for_instance(cfg)
    assert c.operand_path == _capi.OPERAND_LDS
    assert gemm.mapping_report(cfg, c, info).not_honoured["operand_path"] == {
        "requested": "direct_ab", "kernel": "lds"}
    # byte operands have no such kernel; M, N in 16-row blocks; packed operands
    for args, kw in (((128, 256, 512, "fp8_e4m3", "bf16"), {}), ((120, 256, 512, "bf16", "bf16"), {}),
                     ((128, 264, 512, "bf16", "bf16"), {}), ((128, 256, 528, "bf16", "bf16"), {}),
                     ((128, 256, 512, "bf16", "bf16"), dict(lda=520)),
                     ((128, 256, 512, "bf16", "bf16"), dict(ldb=520))):
        with pytest.raises(_capi.AsterGemmError):
            gemm.GemmPlan.create(*args, operand_path="direct_ab", **kw)


def test_repeated_selection_is_remembered_per_config():
    # the library remembers a thread's last selections; a config that differs in any field is a
    # different entry, refusals are never remembered, and more configs than the memory holds
    # still select correctly
    lib = _capi.load()
    names = {}
    shapes = [(256 * i, 1024 * j, 2048 * j) for i in range(1, 6) for j in range(1, 6)]   # 25 > 16 entries
    for rnd in range(3):
        for shape in shapes:
            for dt in ("bf16", "fp8_e4m3"):
                name = gemm.GemmPlan.create(*shape, dt, "bf16").info.name.decode()
                assert names.setdefault((shape, dt), name) == name
    assert len(set(names.values())) >= 3, set(names.values())
    for _ in range(2):
        with pytest.raises(_capi.AsterGemmError) as err:
            gemm.GemmPlan.create(120, 256, 512, "bf16", "bf16", operand_path="direct_ab")
        assert "M % 16" in str(err.value)
    a = gemm.GemmPlan.create(16, 14336, 4096, "bf16", "bf16")
    b = gemm.GemmPlan.create(16, 14336, 4096, "bf16", "f32")
    c = gemm.GemmPlan.create(16, 14336, 4096, "bf16", "bf16", has_bias=True)
    assert a.info.name != b.info.name and a.info.name == c.info.name
    assert lib.astergemm_variant_count() > 0


def test_selection_from_many_threads_is_consistent():
    # the selection memory is per thread: threads that select different configs at the same time
    # never see each other's entries
    import threading
    shapes = [(256 * (i + 1), 1024 * (i % 3 + 1), 2048 * (i % 2 + 1)) for i in range(8)]
    want = [gemm.GemmPlan.create(*s_, "bf16", "bf16").info.name for s_ in shapes]
    bad = []

    def worker(i):
        for _ in range(300):
            for j in (i, (i + 3) % 8):
                name = gemm.GemmPlan.create(*shapes[j], "bf16", "bf16").info.name
                if name != want[j]:
                    bad.append((i, j, name))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not bad, bad[:3]


def test_execute_checks_host_operand_sizes_before_touching_the_gpu(tmp_path):
    cfg = make_instance(256, 256, 256)
    path, _ = gemm.compile_gemm(cfg, str(tmp_path / "k.hsaco"))
    A = np.zeros((256, 256), np.uint16)
    B = np.zeros((256, 256), np.uint16)
    # (no GPU here: any of these would fail in hip_init if the check came later)
    with pytest.raises(ValueError, match="A holds"):
        gemm.execute_gemm_hsaco(cfg, path, 1, A[:128], B, skip_gpu_check=True)
    with pytest.raises(ValueError, match="B holds"):
        gemm.execute_gemm_hsaco(cfg, path, 1, A, np.zeros((256, 128), np.uint16), skip_gpu_check=True)
    with pytest.raises(ValueError, match="storage type"):
        gemm.execute_gemm_hsaco(cfg, path, 1, A.view(np.uint8), B, skip_gpu_check=True)
    with pytest.raises(ValueError, match="storage type"):
        gemm.execute_gemm_hsaco(cfg, path, 1, A.astype(np.float32), B, skip_gpu_check=True)
    q = make_instance(256, 256, 256, dtype_ab="mxfp4")
    a4 = np.zeros((256, 128), np.uint8)
    mx = np.full((256, 8), 127, np.uint8)
    with pytest.raises(ValueError, match="mx_a is required"):
        gemm.check_host_operands(q, a4, a4)
    with pytest.raises(ValueError, match="mx_b must be"):
        gemm.check_host_operands(q, a4, a4, mx_a=mx, mx_b=mx[:, :4])
    gemm.check_host_operands(q, a4, a4, mx_a=mx, mx_b=mx)
    b = make_instance(256, 256, 256, has_bias=True)
    with pytest.raises(ValueError, match="bias"):
        gemm.check_host_operands(b, A, B, bias=np.zeros(255, np.float32))


def test_workspace_query_and_caller_workspace_checks():
    # shapes that are not cut into K ranges need no workspace
    assert gemm.GemmPlan.create(8192, 8192, 8192).workspace_bytes() == 0
    assert gemm.GemmPlan.create(16, 14336, 4096).workspace_bytes() == 0
    # split K on the 128 x 128 kernel: 8 ranges of 128 x 4096 fp32 partial sums
    p = gemm.GemmPlan.create(128, 4096, 14336)
    assert p.info.name.decode().startswith("splitk_") and p.workspace_bytes() == 8 * 128 * 4096 * 4
    assert p.workspace_bytes() == _capi.NOALLOC_SCRATCH_BYTES
    # decode rows of 28 KiB: 7 ranges of 4 KiB
    d = gemm.GemmPlan.create(16, 4096, 14336)
    assert d.workspace_bytes() == 7 * 16 * 4096 * 4
    # a workspace that is too small, or misaligned, is refused before anything is launched
    with pytest.raises(_capi.AsterGemmError, match="workspace of"):
        d.run(4096, 4096, 4096, workspace=4096, workspace_bytes=d.workspace_bytes() - 1)
    with pytest.raises(_capi.AsterGemmError, match="dWorkspace must be 16-byte aligned"):
        d.run(4096, 4096, 4096, workspace=4096 + 4, workspace_bytes=d.workspace_bytes())
    # the entry point that allocates nothing refuses what its scratch cannot hold
    big = gemm.GemmPlan.create(512, 4096, 14336)
    assert big.workspace_bytes() > _capi.NOALLOC_SCRATCH_BYTES
    with pytest.raises(_capi.AsterGemmError, match="built-in scratch"):
        big.run_noalloc(4096, 4096, 4096)
    with pytest.raises(_capi.AsterGemmError, match="non-null"):
        gemm.GemmPlan.create(256, 256, 256).run_noalloc(None, None, None)


def test_reported_grid_is_the_launched_grid_of_the_k_range_kernels():
    # S K ranges x R row ranges, one workgroup per CU: the description comes from the same
    # function the launcher uses (the number of CUs is 0 without a device: one row range)
    def krange_grid(mh, N, S, cus):
        slots = (cus // 16) * 8 if mh == 2 else cus
        rows = min(max(slots // S, 1), (N + 15) // 16)
        g = mh * S * rows
        return (g + 15) // 16 * 16 if mh == 2 else g

    # (M, N, K, K ranges, workgroups per row range): over 32 rows one workgroup covers all
    # activation rows (four tiles per wave on 4 KiB ranges) except on rows of exactly 8 KiB or of
    # more than 16 such ranges, which keep two workgroups per row range
    for (M, N, K, S, mh) in ((16, 4096, 14336, 7, 1), (16, 4096, 28672, 7, 1), (64, 4096, 14336, 7, 1),
                             (16, 8192, 28672, 7, 1), (64, 14336, 4096, 1, 2), (33, 520, 2048, 1, 1),
                             (64, 14336, 8192, 4, 1), (64, 512, 3072, 2, 1), (64, 4096, 40960, 10, 2)):
        p = gemm.GemmPlan.create(M, N, K, family=_capi.KERNEL_SKINNY)
        assert p.info.name.decode().startswith("skinnyx_bf16_m64")
        assert p.workspace_bytes() == (S * M * N * 4 if S > 1 else 0)
        assert p.info.grid_x == krange_grid(mh, N, S, cus=0)


def test_runtime_seam_function_free_and_cluster_launch():
    lib = _capi.load()
    assert lib.aster_rt_function_free(None) == 0
    # a cluster larger than (1,1,1) is refused on gfx950 before the function handle is used
    rc = lib.aster_rt_module_launch_kernel_ex(None, 1, 1, 1, 64, 1, 1, 2, 1, 1, 0, None, None)
    assert rc == -95 and "cluster launch" in _capi.last_error()


# ---- array roles and kernel-argument packing (reference:
# test/integration/test_execution_core.py:51-189) ---------------------------------

def test_array_role_wrappers():
    a = np.zeros(4, np.float32)
    assert InputArray(a).array is a and OutputArray(a).array is a and InOutArray(a).array is a
    assert len({InputArray, OutputArray, InOutArray}) == 3
    assert create_kernel_args_capsule is create_kernel_args


def test_kernel_args_packing():
    assert create_kernel_args() == (None, None, None)
    ptrs, packed, _ = create_kernel_args(7, -3, 1.5, np.int64(9), np.float64(2.25),
                                         ctypes.c_int64(1 << 40), ctypes.c_void_p(0x1234))
    kinds = [t for _, t in packed._fields_]
    assert kinds == [ctypes.c_int32, ctypes.c_int32, ctypes.c_float, ctypes.c_int32, ctypes.c_float,
                     ctypes.c_int64, ctypes.c_void_p]
    assert (packed._field0, packed._field1, packed._field2) == (7, -3, 1.5)
    assert packed._field3 == 9 and packed._field4 == 2.25 and packed._field5 == 1 << 40
    base, size = ctypes.addressof(packed), ctypes.sizeof(packed)
    assert all(base <= p < base + size for p in ptrs)
    arr = np.arange(4, dtype=np.float32)
    ptrs, packed, _ = create_kernel_args(arr)
    assert packed._field0 == arr.ctypes.data
    with pytest.raises(TypeError, match="unsupported argument type"):
        create_kernel_args("nope")


# ---- bench statistics (reference: bench_harness.py:44-90, 174-198) ----------------

def test_init_array_modes_are_deterministic():
    a = BH.init_array((4, 8), "hpl", "A")
    b = BH.init_array((4, 8), BH.InitMode.HPL, "B")
    assert a.dtype == np.float16 and a.shape == (4, 8)
    assert np.array_equal(a.reshape(-1), np.random.default_rng(42).uniform(-0.5, 0.5, 32).astype(np.float16))
    assert np.array_equal(b.reshape(-1), np.random.default_rng(43).uniform(-0.5, 0.5, 32).astype(np.float16))
    t = BH.init_array((8,), "trig_float", "B")
    assert np.array_equal(t, np.cos(np.arange(8, dtype=np.float64)).astype(np.float16))
    assert set(np.unique(BH.init_array((64,), "rand_int", "A")).tolist()) <= {-2, -1, 0, 1, 2}
    assert not BH.init_array((4,), "zero", "A").any()
    assert BH.init_array((2,), "special", "A")[0] == np.float16(65280.0)
    assert BH.init_array((2,), "special", "B")[0] == np.float16(6.07967376708984375e-5)
    n = BH.init_array((16,), "norm_dist", "A", dtype=np.float32)
    assert np.array_equal(n, np.random.default_rng(42).standard_normal(16).astype(np.float32))
    with pytest.raises(ValueError):
        BH.init_array((2,), "nope", "A")
    assert str(BH.INIT_DEFAULT) == "hpl" and BH.NUM_ITERATIONS == 100 and BH.WARMUP_ITERATIONS == 20


def test_percentiles_and_stats():
    times = [float(t) for t in range(100, 200)]          # 100 samples, ns
    assert BH._percentile_ns(times, 0) == 100 and BH._percentile_ns(times, 100) == 199
    assert BH._percentile_ns(times, 50) == 150 and BH._percentile_ns(times, 10) == 110
    s = BH._compute_stats(list(reversed(times)), total_flops=3_000_000, peak_tflops=2500.0)
    assert (s.p0_ns, s.p10_ns, s.p25_ns, s.p50_ns, s.p90_ns) == (100, 110, 125, 150, 189)
    assert s.mean_ns == 149.5 and s.p50_tf == 3_000_000 / 150 * 1e-3
    assert s.p50_pct == s.p50_tf / 2500.0 * 100 and s.p0_ms == 1e-4
    assert BH._compute_stats([], 1, 1.0) is None and BH._compute_stats([5, 0], 1, 1.0) is None
    one = BH._compute_stats([10], 1000, 1.0)
    assert one.stddev_ns == 0.0 and one.stddev_tf == 0.0
    assert BH.peak_tflops_f16("gfx950") == 2500.0 and BH.peak_tflops_f16("gfx942") == 1307.0
    assert BH.peak_tflops("gfx950", "fp8_e4m3") == 5000.0


def test_result_line_roundtrip():
    cfg = make_instance(512, 512, 256)
    s = BH._compute_stats([1000.0, 1100.0, 900.0], cfg.total_flops, 2500.0)
    buf = io.StringIO()
    BH.emit_one_result(buf, "bench_gemm", cfg, s)
    BH.emit_one_result(None, "bench_gemm", cfg, s)
    line = buf.getvalue()
    assert line.startswith("BENCH_RESULT_JSON:")
    rec, = BH.parse_result_lines(["noise", "x " + line, "BENCH_RESULT_JSON:{bad"])
    assert rec["label"] == cfg.label and rec["mcpu"] == "gfx950" and rec["M"] == 512
    assert rec["tflops_median"] == s.p50_tf and rec["sample_n"] == 1
    assert set(rec) == {"mcpu", "bench", "M", "N", "K", "label", "tflops_median", "tflops_p10",
                        "tflops_p90", "tflops_mean", "tflops_p0", "tflops_p25", "tflops_stddev",
                        "pct_peak_p50", "sample_n"}


def test_make_inputs_storage_types():
    cfg = make_instance(256, 256, 64, dtype_ab="bf16")
    a, b = BH.make_inputs(cfg)
    assert a.dtype == np.uint16 and a.shape == (256, 64) and b.shape == (256, 64)
    from oracle import formats as F
    want = F.f32_to_bf16_bits(BH.init_array((256, 64), "hpl", "A").astype(np.float32))
    assert np.array_equal(a, want)


def test_build_scan_finds_a_register_copy_in_front_of_an_inline_asm_mfma():
    # the compiler's hazard recogniser does not look inside inline asm; the build scans the device
    # assembly instead (aster_amd/build.py: scan_mfma_hazards)
    from aster_amd.build import scan_mfma_hazards
    mfma = ("\t;;#ASMSTART\n{pre}\tv_mfma_scale_f32_16x16x128_f8f6f4 a[36:39], v[68:71], v[36:39], a[36:39], "
            "v32, v95 op_sel_hi:[0,0,0] cbsz:4 blgp:4\n\t;;#ASMEND\n")
    copy = "\tv_mov_b64_e32 v[38:39], v[36:37]\n\tv_mov_b64_e32 v[36:37], v[34:35]\n"
    found = scan_mfma_hazards(copy + mfma.format(pre=""))
    assert sorted((f[0], f[2]) for f in found) == [(4, 1), (4, 2)]
    # two wait states in between, of any kind, are enough
    assert scan_mfma_hazards(copy + mfma.format(pre="\ts_nop 1\n")) == []
    assert scan_mfma_hazards(copy + "\ts_add_u32 s0, s1, s2\n\ts_nop 0\n" + mfma.format(pre="")) == []
    # scale and accumulator registers count as sources; other registers do not
    assert len(scan_mfma_hazards("\tv_and_b32_e32 v95, 0xffff, v95\n" + mfma.format(pre=""))) == 1
    assert len(scan_mfma_hazards("\tv_accvgpr_mov_b32 a37, a5\n" + mfma.format(pre=""))) == 1
    assert scan_mfma_hazards("\tv_mov_b32_e32 v40, v41\n" + mfma.format(pre="")) == []
    # MFMAs the compiler emitted itself are its own business
    assert scan_mfma_hazards(copy + "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[36:39], v[4:7], a[0:3]\n") == []
    # a spilled scalar base restored by v_readlane right in front of an inline-asm transfer
    g2s = ("\t;;#ASMSTART\n\ts_mov_b32 m0, s12\n\ts_nop 0\n\tglobal_load_lds_dwordx4 v9, s[4:5]\n"
           "\t;;#ASMEND\n")
    assert len(scan_mfma_hazards("\tv_readlane_b32 s4, v127, 3\n\tv_readlane_b32 s5, v127, 4\n" + g2s)) == 2
    assert scan_mfma_hazards("\tv_readlane_b32 s4, v127, 3\n\ts_nop 3\n" + g2s) == []
    assert scan_mfma_hazards("\ts_add_u32 s4, s6, s7\n" + g2s) == []


def test_build_scan_follows_the_back_edge_of_a_loop():
    # a VALU write at the bottom of a loop and an inline-asm MFMA at its head are neighbours in
    # execution order although the text has them far apart
    from aster_amd.build import scan_mfma_hazards
    mfma = ("\t;;#ASMSTART\n\tv_mfma_f32_16x16x32_bf16 a[0:3], v[36:39], v[4:7], a[0:3]\n\t;;#ASMEND\n")
    filler = "\ts_add_u32 s0, s1, s2\n" * 6
    loop = ("kern:                                   ; @kern\n" + filler + ".LBB0_1:    ; =>This Inner Loop\n" + mfma +
            filler + "\tv_mov_b32_e32 v5, v9\n\ts_cbranch_scc1 .LBB0_1\n" + "\ts_endpgm\n")
    found = scan_mfma_hazards(loop)
    assert len(found) == 1 and "v_mov_b32_e32 v5" in found[0][3]
    # the branch itself is one wait state: one more instruction in between is enough
    ok = loop.replace("\tv_mov_b32_e32 v5, v9\n", "\tv_mov_b32_e32 v5, v9\n\ts_nop 0\n")
    assert scan_mfma_hazards(ok) == []
    # a forward branch over the wait states brings the write next to the MFMA as well
    skip = ("kern:\n\tv_mov_b32_e32 v5, v9\n\ts_cbranch_scc1 .LBB0_2\n" + filler + ".LBB0_2:\n" + mfma)
    assert len(scan_mfma_hazards(skip)) == 1
    # nothing falls through an unconditional branch
    dead = ("kern:\n\ts_branch .LBB0_3\n\tv_mov_b32_e32 v5, v9\n.LBB0_3:\n" + mfma)
    assert scan_mfma_hazards(dead) == []


def test_spills_beside_hand_counted_loads_are_found():
    # a kernel that loads registers in inline assembly counts those loads itself; the compiler,
    # which inserts no wait for them, must not spill in such a kernel (aster_amd/asm_scan.py)
    from aster_amd.build import scan_spills_beside_asm_loads
    load = "\t;;#ASMSTART\n\tbuffer_load_dwordx4 v[8:11], v123, s[16:19], s66 offen\n\t;;#ASMEND\n"
    lds = "\t;;#ASMSTART\n\tglobal_load_lds_dwordx4 v98, s[56:57]\n\t;;#ASMEND\n"
    spill = "\tscratch_store_dwordx4 off, v[8:11], off ; 16-byte Folded Spill\n"
    assert scan_spills_beside_asm_loads("k1:\n" + load + spill) == [("k1", 1)]
    # function labels as the compiler writes them, with a trailing comment
    assert scan_spills_beside_asm_loads("k1:        ; @k1\n" + load + spill) == [("k1", 1)]
    assert scan_spills_beside_asm_loads("k1:\n" + load + "k2:\n" + spill) == []
    assert scan_spills_beside_asm_loads("k1:\n" + lds + spill) == []       # transfers into LDS write no register
    assert scan_spills_beside_asm_loads("k1:\n.LBB0_1:\n" + load + ".LBB0_2:\n" + spill + spill) == [("k1", 2)]
    assert scan_spills_beside_asm_loads("k1:\n\tbuffer_load_dwordx4 v[8:11], v1, s[0:3], 0 offen\n" + spill) == []
    # gfx950 spills vector registers into accumulation registers first: a copy of a register that
    # an inline-asm load writes counts, a copy of any other register does not
    assert scan_spills_beside_asm_loads("k1:\n" + load + "\tv_accvgpr_write_b32 a200, v9\n") == [("k1", 1)]
    assert scan_spills_beside_asm_loads("k1:\n" + load + "\tv_accvgpr_write_b32 a200, v12\n") == []
    assert scan_spills_beside_asm_loads("k1:\n" + load + "\tv_accvgpr_write_b32 a0, 0\n") == []
    # and the allocator's own account in the kernel metadata
    meta = ("\t.amdgpu_metadata\n---\namdhsa.kernels:\n  - .agpr_count:     0\n    .args:\n"
            "      - .name:           p\n        .size: 8\n    .name:           {name}\n"
            "    .sgpr_spill_count: {s}\n    .symbol:         {name}.kd\n    .vgpr_spill_count: {v}\n"
            "...\n\t.end_amdgpu_metadata\n")
    assert scan_spills_beside_asm_loads("k1:\n" + load + meta.format(name="k1", s=0, v=0)) == []
    assert scan_spills_beside_asm_loads("k1:\n" + load + meta.format(name="k1", s=3, v=1)) == [("k1", 4)]
    assert scan_spills_beside_asm_loads("k1:\n" + load + meta.format(name="k2", s=3, v=1)) == []


def test_direct_b_loads_of_edge_tiles_stay_inside_the_payload():
    # The pre-shuffled-B stream kernels address B as buffer resource + scalar offset (16-row block
    # and K-step) + lane offset (+ 1 KiB immediate); the hardware checks only the lane offset and
    # the immediate against the resource, so the scalar part must never leave the payload.  This
    # models the offset arithmetic of gemm_stream8db / gemm_stream4db / gemm_streamdb_kernel.hpp
    # (block index clamped to the last block of B) over edge shapes.
    def extent(N, K, bytes_per_k_num, bytes_per_k_den, group, clamp):
        row_bytes = K * bytes_per_k_num // bytes_per_k_den
        chunk_row = 16 * row_bytes                     # bytes of a 16-row block
        steps_bytes = row_bytes * 16                   # a block's K-steps lie back to back
        worst = 0
        for col0 in range(0, N, 256):
            for wn in range(4):
                for n in range(4):
                    nb = (col0 >> 4) + wn * 4 + n
                    if clamp:
                        nb = min(nb, (N >> 4) - 1)
                    worst = max(worst, nb * chunk_row + steps_bytes)   # one past the block's last byte
        return worst
    for N in (16, 64, 80, 192, 272, 1000 // 16 * 16, 4096 + 64):
        for K in (128, 512, 4096):
            payload = N * K                               # fp8: one byte per element
            assert extent(N, K, 1, 1, 16, clamp=True) <= payload
            if N % 256:
                assert extent(N, K, 1, 1, 16, clamp=False) > payload   # what the clamp is for
    for N in (64, 128, 192, 320, 4096 + 64):
        for K in (512, 4096):
            payload = N * K // 2
            assert extent(N, K, 1, 2, 16, clamp=True) <= payload
            # lane-order scale plane: 64-row groups of (K / 256) * 512 bytes
            groups = N >> 6
            plane = groups * (K // 256) * 512
            worst = max(min((col0 >> 6) + wn, groups - 1) + 1 for col0 in range(0, N, 256) for wn in range(4))
            assert worst * (K // 256) * 512 <= plane


def test_library_and_pytorch_share_one_hip_runtime_whichever_loads_first():
    """Loading the library before `import torch` must not leave two copies of the HIP runtime
    in the process: the one initialised second finds no device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("from aster_amd import _capi; _capi.load(); import torch\n"
            "for name in ('libamdhip64', 'libhsa-runtime64'):\n"
            "    paths = {l.split()[-1] for l in open('/proc/self/maps') if name in l}\n"
            "    assert len(paths) == 1, paths\n"
            "print('one runtime')\n")
    out = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "one runtime" in out.stdout, out.stderr[-2000:]
