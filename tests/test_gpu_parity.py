"""GPU parity: the HIP kernels, called through the C-ABI, against the CPU oracle on
the same seeded inputs.

Bars: rel-L2 <= 1e-3 against the fp32-accumulated oracle for every floating
output (bf16 / f16 outputs are compared with the oracle's output rounded the
same way); the reference's own bar `assert_allclose(rtol=1e-2, atol=1e-2)` on
its own test shapes; bit-exact where the arithmetic is exact (known answers,
power-of-two scaling, identity operand, run-to-run determinism).
"""
import ctypes
import json
import os

import numpy as np
import pytest

from aster_amd import _capi, gemm as AG
from aster_amd.execution import GpuBuffer
from aster_amd.gemm_config import (Cdna4GemmInstance, GemmMappingSpec, GemmSpec, OperandPath,
                                   make_instance)
from oracle import cgemm, formats as F, gemm as G

pytestmark = pytest.mark.gpu

REL_L2_BAR = 1e-3
_DT = {"f16": G.F16, "bf16": G.BF16, "fp8_e4m3": G.FP8_E4M3, "mxfp4": G.MXFP4, "f32": G.F32}
_OUT_NP = {"f32": np.float32, "bf16": np.uint16, "f16": np.uint16}


def run_gemm(a, b, M, N, K, dtype_ab, dtype_c, *, scale_a=None, scale_b=None, mx_a=None, mx_b=None,
             bias=None, lda=0, ldb=0, ldc=0, family=_capi.KERNEL_AUTO, wg_tile=(0, 0),
             operand_path="lds", variant=0, mx_a_layout="rows"):
    """Upload, launch once through astergemm_run, download.  Returns the raw
    output storage [M, ldc or N] and the kernel name."""
    plan = AG.GemmPlan.create(M, N, K, dtype_ab, dtype_c, has_bias=bias is not None, lda=lda,
                              ldb=ldb, ldc=ldc, family=family, wg_tile=wg_tile,
                              operand_path=operand_path, variant=variant, mx_a_layout=mx_a_layout)
    ldc_eff = ldc or N
    out = np.full((M, ldc_eff), 0x7FC1 if dtype_c != "f32" else np.nan, dtype=_OUT_NP[dtype_c])
    bufs = []

    def up(x):
        if x is None:
            return None
        x = np.ascontiguousarray(x)
        buf = GpuBuffer(x.nbytes)
        buf.copy_from_host(x)
        bufs.append(buf)
        return buf.ptr_value

    dA, dB, dC = up(a), up(b), up(out)
    kw = {}
    if scale_a is not None:
        kw["scale_a"] = up(np.array([scale_a], np.float32))
        kw["scale_b"] = up(np.array([scale_b], np.float32))
    if mx_a is not None:
        kw["mx_a"], kw["mx_b"] = up(mx_a), up(mx_b)
    if bias is not None:
        kw["bias"] = up(np.asarray(bias, np.float32))
    print(f"launch {plan.info.name.decode()} M={M} N={N} K={K}", flush=True)
    plan.run(dA, dB, dC, **kw)
    bufs[2].copy_to_host(out)
    for bf in bufs:
        bf.free()
    return out, plan.info.name.decode()


def check(out_raw, want_raw, dtype_c, N, bar=REL_L2_BAR):
    got = G.output_to_f32(out_raw[:, :N], _DT[dtype_c])
    want = G.output_to_f32(want_raw, _DT[dtype_c])
    assert not np.isnan(got).any()
    rel = G.rel_l2(got, want)
    assert rel <= bar, f"rel-L2 {rel:.3e} > {bar}"
    return rel


def operands(M, N, K, dtype_ab, seed=42, a_std=1.0, b_std=0.02, dist="normal"):
    """Seeded operands in storage form: seeds `seed` (A) and `seed + 1` (B)."""
    ra, rb = np.random.default_rng(seed), np.random.default_rng(seed + 1)
    if dist == "uniform":
        xa = ra.uniform(-1, 1, (M, K)).astype(np.float32)
        xb = rb.uniform(-1, 1, (N, K)).astype(np.float32)
    else:
        xa = (ra.standard_normal((M, K)) * a_std).astype(np.float32)
        xb = (rb.standard_normal((N, K)) * b_std).astype(np.float32)
    extra = {}
    if dtype_ab == "f16":
        a, b = xa.astype(np.float16), xb.astype(np.float16)
    elif dtype_ab == "bf16":
        a, b = F.f32_to_bf16_bits(xa), F.f32_to_bf16_bits(xb)
    elif dtype_ab == "fp8_e4m3":
        a, sa = F.quantize_fp8_tensor(xa)
        b, sb = F.quantize_fp8_tensor(xb)
        extra = dict(scale_a=sa, scale_b=sb)
    else:
        a, mxa = F.quantize_mxfp4(xa)
        b, mxb = F.quantize_mxfp4(xb)
        extra = dict(mx_a=mxa, mx_b=mxb)
    return a, b, extra


# ---- configuration 1 of the baseline: fp16 256^3, uniform[-1,1], fp32 out ---------

def test_config1_fp16_256(gpu):
    a, b, _ = operands(256, 256, 256, "f16", dist="uniform")
    out, _ = run_gemm(a, b, 256, 256, 256, "f16", "f32")
    want = G.gemm(a, b, G.F16, G.F32)
    check(out, want, "f32", 256)
    assert G.rel_l2(out, cgemm.gemm_raw(a, b, G.F16, 256, 256, 256)) <= REL_L2_BAR
    np.testing.assert_allclose(out, want, rtol=1e-2, atol=1e-2)


# ---- the reference's own GEMM test shapes (f16 x f16 -> f32) -------------------------
# TestCdna4GemmG2S / MultiWG / Coop8Waves / Pipelined8Wave of
# contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:493-570:
# M = wg_m * twg_m * 16, N = wg_n * twg_n * 16, K = 32 * k_mult,
# inputs np.random.seed(42 + M + N + K); randn * 0.1 -> f16.
REFERENCE_SHAPES = (
    [((1, 1), twg, km) for twg in ((2, 2), (2, 1), (1, 2)) for km in (1, 2, 4, 8)]
    + [((2, 2), (2, 2), 4)]
    + [((1, 1), twg, 4) for twg in ((4, 16), (16, 4), (2, 32), (32, 2))]
    + [((1, 1), (8, 8), 8), ((1, 1), (8, 8), 5)]
)


@pytest.mark.parametrize("wg,twg,k_mult", REFERENCE_SHAPES)
def test_reference_test_shapes_f16(gpu, wg, twg, k_mult):
    M, N, K = wg[0] * twg[0] * 16, wg[1] * twg[1] * 16, 32 * k_mult
    np.random.seed(42 + M + N + K)
    a = (np.random.randn(M, K) * 0.1).astype(np.float16)
    b = (np.random.randn(N, K) * 0.1).astype(np.float16)
    spec = GemmSpec.from_sizes(M, N, K, mfma_shape=[16, 16, 32])
    mapping = GemmMappingSpec([wg[0], wg[1], 1], [1, 1, 1], [twg[0], twg[1], 1],
                              operand_path=OperandPath.DIRECT_B, mcpu="gfx950")
    cfg = Cdna4GemmInstance(spec, mapping)
    import tempfile
    with tempfile.NamedTemporaryFile(suffix=".hsaco") as tmp:
        AG.compile_gemm(cfg, tmp.name)
        c_flat, times = AG.execute_gemm_hsaco(cfg, tmp.name, 1, a, b)
    expected = (a.astype(np.float32) @ b.astype(np.float32).T).flatten()
    np.testing.assert_allclose(c_flat, expected, rtol=1e-2, atol=1e-2)   # the reference's bar
    assert G.rel_l2(c_flat, expected) <= REL_L2_BAR                      # this build's bar
    assert len(times) == 1 and times[0] > 0
    # the same problem through the LDS-staged tile kernel
    out, name = run_gemm(a, b, M, N, K, "f16", "f32", family=_capi.KERNEL_TILE)
    assert name.startswith("tile")
    np.testing.assert_allclose(out.flatten(), expected, rtol=1e-2, atol=1e-2)
    assert G.rel_l2(out.flatten(), expected) <= REL_L2_BAR


# ---- scaled-down versions of configurations 2-5, same distributions and seeds --------

@pytest.mark.parametrize("M,N,K,tile", [(512, 512, 512, 256), (384, 640, 448, 128), (256, 256, 64, 128)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_config2_bf16(gpu, M, N, K, tile, dtype_c):
    a, b, _ = operands(M, N, K, "bf16")
    out, name = run_gemm(a, b, M, N, K, "bf16", dtype_c, family=_capi.KERNEL_TILE, wg_tile=(tile, tile))
    assert f"{tile}x{tile}" in name
    check(out, G.gemm(a, b, G.BF16, _DT[dtype_c]), dtype_c, N)


@pytest.mark.parametrize("M,N,K,tile", [(512, 512, 512, 256), (256, 384, 640, 128)])
def test_config3_fp8_per_tensor_scales(gpu, M, N, K, tile):
    a, b, ex = operands(M, N, K, "fp8_e4m3", a_std=1.0, b_std=1.0)
    out, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", "bf16", wg_tile=(tile, tile), **ex)
    want = G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=G.BF16)
    check(out, want, "bf16", N)
    # against the float64-accumulated product: the fp8 matrix-core path sums each
    # 128-wide block of products in a fixed-point adder tree that is a little
    # narrower than fp32 (measured rel-L2 ~1.3e-5 on fp32 outputs), so a handful
    # of bf16 outputs land 2 ulp away; none further.
    w64 = G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=G.BF16, accumulate="f64")
    # (entries that cancel to almost nothing are judged by rel-L2 above, not in ulps)
    w64f = F.bf16_bits_to_f32(w64)
    solid = np.abs(w64f) > 1e-2 * np.sqrt(np.mean(w64f.astype(np.float64) ** 2))
    ulp = np.abs(out.astype(np.int32) - w64.astype(np.int32))
    assert ulp[solid].max() <= 2 and np.mean(ulp[solid] > 1) < 1e-3
    out32, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", wg_tile=(tile, tile), **ex)
    check(out32, G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=G.F32), "f32", N, bar=1e-4)


@pytest.mark.parametrize("M,N,K,tile", [(512, 512, 512, 256), (256, 384, 768, 128)])
def test_config5_mxfp4(gpu, M, N, K, tile):
    a, b, ex = operands(M, N, K, "mxfp4", a_std=1.0, b_std=1.0)
    out, _ = run_gemm(a, b, M, N, K, "mxfp4", "bf16", wg_tile=(tile, tile), **ex)
    check(out, G.gemm_mxfp4(a, ex["mx_a"], b, ex["mx_b"], out_dtype=G.BF16), "bf16", N)
    out32, _ = run_gemm(a, b, M, N, K, "mxfp4", "f32", wg_tile=(tile, tile), **ex)
    check(out32, G.gemm_mxfp4(a, ex["mx_a"], b, ex["mx_b"], out_dtype=G.F32), "f32", N, bar=1e-5)


def test_mxfp4_nonuniform_scales_pin_the_lane_to_k_block_mapping(gpu):
    # every (row, K-block) gets its own e8m0 byte and every element its own code:
    # a wrong lane <-> K-block pairing cannot cancel.
    M = N = 128
    K = 512
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (M, K // 2)).astype(np.uint8)
    b = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    mxa = rng.integers(118, 134, (M, K // 32)).astype(np.uint8)
    mxb = rng.integers(118, 134, (N, K // 32)).astype(np.uint8)
    out, _ = run_gemm(a, b, M, N, K, "mxfp4", "f32", mx_a=mxa, mx_b=mxb)
    check(out, G.gemm_mxfp4(a, mxa, b, mxb, out_dtype=G.F32), "f32", N, bar=1e-5)


@pytest.mark.parametrize("M", [1, 16, 64])
def test_config4_skinny_full_size(gpu, M):
    N, K = 14336, 4096
    a, b, _ = operands(M, N, K, "bf16", a_std=1.0, b_std=0.02)
    out, name = run_gemm(a, b, M, N, K, "bf16", "bf16")
    assert name.startswith("skinny")
    check(out, G.gemm(a, b, G.BF16, G.BF16), "bf16", N)


@pytest.mark.parametrize("M,N,K", [(3, 100, 64), (17, 264, 1056), (33, 48, 32), (64, 1032, 4096)])
@pytest.mark.parametrize("dtype_ab", ["bf16", "f16"])
def test_skinny_ragged(gpu, M, N, K, dtype_ab):
    a, b, _ = operands(M, N, K, dtype_ab, seed=7, b_std=0.05)
    bias = np.random.default_rng(9).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, dtype_ab, "f32", bias=bias)
    assert name.startswith("skinny")
    check(out, G.gemm(a, b, _DT[dtype_ab], G.F32, bias=bias), "f32", N, bar=1e-5)


@pytest.mark.parametrize("M,N,K", [(16, 14337, 4096), (1, 8, 2048), (5, 777, 8192), (13, 6000, 2048),
                                   (16, 24, 4096), (9, 4104, 8192), (16, 40, 2048)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "f32"), ("f16", "f16"), ("bf16", "bf16")])
def test_skinny_resident_activations(gpu, M, N, K, dtype_ab, dtype_c):
    """M <= 16 and K in {2048, 4096, 8192} take the persistent kernel that keeps x in
    registers; row ranges that end inside a 16-row block, single-workgroup grids,
    bias and a padded output pitch."""
    a, b, _ = operands(M, N, K, dtype_ab, seed=11, b_std=0.05)
    bias = np.random.default_rng(12).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc)
    assert name.startswith("skinnyx")
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
    check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    # the pad columns of every output row stay untouched
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(64, 14336, 4096), (17, 8, 2048), (32, 777, 4096), (33, 6000, 2048),
                                   (50, 24, 4096), (64, 14337, 2048), (48, 4104, 4096), (64, 136, 4096)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "f32"), ("f16", "f16"), ("bf16", "bf16")])
def test_skinny_resident_activations_up_to_64_rows(gpu, M, N, K, dtype_ab, dtype_c):
    """16 < M <= 64 with K in {2048, 4096}: two activation tiles per wave; above 32 rows four
    tiles per wave on 4 KiB rows, and two workgroups per row range (one half of the activation
    rows each) on 8 KiB rows."""
    a, b, _ = operands(M, N, K, dtype_ab, seed=61, b_std=0.05)
    bias = np.random.default_rng(62).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc)
    assert name.startswith("skinnyx") and "_m64_" in name
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
    check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(16, 4096, 14336), (1, 8, 6144), (33, 777, 14336), (64, 4096, 14336),
                                   (16, 1000, 28672), (64, 24, 10240), (7, 4104, 32768), (40, 2050, 12288),
                                   (16, 4096, 11008), (16, 5120, 13824), (33, 100, 2304), (64, 520, 6400),
                                   (5, 64, 3840), (40, 136, 40960), (64, 520, 8192)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "f32"), ("f16", "f16"), ("bf16", "bf16")])
def test_skinny_resident_activations_long_rows(gpu, M, N, K, dtype_ab, dtype_c):
    """Rows that are not 4 or 8 KiB (down-projections): the persistent kernel runs one K range
    per workgroup, the last range possibly short, leaves fp32 partial sums in the library's
    workspace and a second kernel adds them in a fixed order; run twice, the results are the
    same bits."""
    a, b, _ = operands(M, N, K, dtype_ab, seed=71, b_std=0.05)
    bias = np.random.default_rng(72).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc, family=_capi.KERNEL_SKINNY)
    assert name.startswith("skinnyx") and "_m64_" in name
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
    check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()
    again, _ = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc, family=_capi.KERNEL_SKINNY)
    assert np.array_equal(out[:, :N].view(np.uint8), again[:, :N].view(np.uint8))


def test_skinny_long_rows_on_two_streams(gpu):
    """Launches in K ranges on two streams at once: each stream has its own partial-sum
    workspace, so interleaved launches give the bits of launches made alone; a larger problem
    on the same stream afterwards grows that stream's workspace."""
    from aster_amd.execution import GpuStream
    shapes = [(16, 4096, 14336), (48, 2048, 11008)]
    streams = [GpuStream(), GpuStream()]
    jobs = []
    for (M, N, K), st in zip(shapes, streams):
        a, b, _ = operands(M, N, K, "bf16", seed=81 + M, b_std=0.05)
        alone, name = run_gemm(a, b, M, N, K, "bf16", "bf16", family=_capi.KERNEL_SKINNY)
        assert "_m64_" in name
        plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16", family=_capi.KERNEL_SKINNY)
        bufs = [GpuBuffer(x.nbytes) for x in (a, b, alone)]
        bufs[0].copy_from_host(np.ascontiguousarray(a))
        bufs[1].copy_from_host(np.ascontiguousarray(b))
        jobs.append((plan, bufs, alone, st))
    for _ in range(8):
        for plan, bufs, _, st in jobs:
            plan.run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2].ptr_value, stream=st.handle.value)
    for plan, bufs, alone, st in jobs:
        st.synchronize()
        got = np.empty_like(alone)
        bufs[2].copy_to_host(got)
        assert np.array_equal(got, alone)
    # the first stream's workspace was sized for 16 x 4096: this one needs more
    M, N, K = 64, 20480, 10240
    a, b, _ = operands(M, N, K, "bf16", seed=83, b_std=0.05)
    alone, _ = run_gemm(a, b, M, N, K, "bf16", "bf16", family=_capi.KERNEL_SKINNY)
    plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16", family=_capi.KERNEL_SKINNY)
    big = [GpuBuffer(x.nbytes) for x in (a, b, alone)]
    big[0].copy_from_host(np.ascontiguousarray(a))
    big[1].copy_from_host(np.ascontiguousarray(b))
    st = streams[0]
    plan.run(big[0].ptr_value, big[1].ptr_value, big[2].ptr_value, stream=st.handle.value)
    st.synchronize()
    got = np.empty_like(alone)
    big[2].copy_to_host(got)
    assert np.array_equal(got, alone)
    for _, bufs, _, _ in jobs:
        for bf in bufs:
            bf.free()
    for bf in big:
        bf.free()
    for st in streams:
        st.destroy()


def test_skinny_long_rows_from_two_host_threads(gpu):
    """Two host threads, a stream each, launching K-range GEMMs at the same time (ctypes drops
    the interpreter lock during the call): the library's per-stream workspaces are handed out
    under a lock, results equal those of launches made alone."""
    import threading
    from aster_amd.execution import GpuStream
    shapes = [(16, 2048, 14336), (33, 1024, 11008)]
    jobs, errors = [], []
    for (M, N, K) in shapes:
        a, b, _ = operands(M, N, K, "bf16", seed=91 + M, b_std=0.05)
        alone, _ = run_gemm(a, b, M, N, K, "bf16", "bf16", family=_capi.KERNEL_SKINNY)
        bufs = [GpuBuffer(x.nbytes) for x in (a, b, alone)]
        bufs[0].copy_from_host(np.ascontiguousarray(a))
        bufs[1].copy_from_host(np.ascontiguousarray(b))
        jobs.append((AG.GemmPlan.create(M, N, K, "bf16", "bf16", family=_capi.KERNEL_SKINNY), bufs, alone))

    def work(plan, bufs):
        try:
            st = GpuStream()
            for _ in range(50):
                plan.run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2].ptr_value, stream=st.handle.value)
            st.synchronize()
            st.destroy()
        except Exception as e:  # surfaced below: an assert in a thread is not seen by pytest
            errors.append(e)

    threads = [threading.Thread(target=work, args=(plan, bufs)) for plan, bufs, _ in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for _, bufs, alone in jobs:
        got = np.empty_like(alone)
        bufs[2].copy_to_host(got)
        assert np.array_equal(got, alone)
        for bf in bufs:
            bf.free()


@pytest.mark.parametrize("M,N,K", [(16, 4096, 14336), (3, 8, 12288), (48, 777, 28672), (64, 4104, 16384),
                                   (16, 520, 11264), (40, 64, 4608)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_skinny_fp8_long_rows(gpu, M, N, K, dtype_c):
    a, b, extra = operands(M, N, K, "fp8_e4m3", seed=75, b_std=0.05)
    bias = np.random.default_rng(76).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias, ldc=N + 8, family=_capi.KERNEL_SKINNY, **extra)
    assert name.startswith("skinnyx_fp8_m64")
    want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-4 if dtype_c == "f32" else REL_L2_BAR)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(16, 14336, 4096), (1, 8, 4096), (5, 777, 8192), (16, 24, 16384),
                                   (13, 6000, 4096), (16, 14337, 8192)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32", "f16"])
def test_skinny_fp8_resident_activations(gpu, M, N, K, dtype_c):
    """fp8 weights through the same persistent kernel (one 16x16x128 MFMA per 128-byte step);
    the result equals the tile kernel's up to fp32 summation order."""
    a, b, extra = operands(M, N, K, "fp8_e4m3", seed=31, b_std=0.05)
    bias = np.random.default_rng(32).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias, ldc=ldc, **extra)
    assert name.startswith("skinnyx_fp8")
    want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-4 if dtype_c == "f32" else REL_L2_BAR)
    else:
        # few outputs: a handful of flipped roundings decide rel-L2, so bound every element by
        # two units in the last place of the 16-bit output (under 1 % above one unit) plus the
        # summation noise of the fp8 MFMA, which matters where the bias cancels the sum
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        ulp = 2.0 ** -7 if dtype_c == "bf16" else 2.0 ** -10
        err = np.abs(got - ref)
        assert np.all(err <= 2 * ulp * np.abs(ref) + 1e-4 * np.abs(ref).max())
        assert np.mean(err > ulp * np.abs(ref) + 1e-4 * np.abs(ref).max()) < 0.01
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()
    if dtype_c == "f32":
        tile, tname = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", bias=bias, family=_capi.KERNEL_TILE,
                               **extra)
        assert not tname.startswith("skinny")
        assert G.rel_l2(out[:, :N], tile) <= 1e-5


@pytest.mark.parametrize("M,N,K", [(64, 14336, 4096), (17, 8, 4096), (33, 777, 8192), (48, 6000, 4096)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_skinny_fp8_up_to_64_rows(gpu, M, N, K, dtype_c):
    a, b, extra = operands(M, N, K, "fp8_e4m3", seed=35, b_std=0.05)
    bias = np.random.default_rng(36).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias, ldc=N + 8, **extra)
    assert name.startswith("skinnyx_fp8_m64")
    want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-4 if dtype_c == "f32" else REL_L2_BAR)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(16, 14336, 4096), (1, 8, 4096), (5, 777, 8192), (16, 24, 16384),
                                   (13, 6000, 4096), (16, 14337, 8192), (9, 1000, 16384)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_skinny_mxfp4_resident_activations(gpu, M, N, K, dtype_c):
    """MXFP4 weights and activations through the persistent kernel: two scaled MFMAs per
    128-byte step, every lane with its own e8m0 byte for both operands."""
    a, b, extra = operands(M, N, K, "mxfp4", seed=41, b_std=0.05)
    # spread the block scales so that a wrong byte cannot go unnoticed
    rng = np.random.default_rng(43)
    extra["mx_a"] = (extra["mx_a"].astype(np.int32) + rng.integers(-3, 4, extra["mx_a"].shape)).astype(np.uint8)
    extra["mx_b"] = (extra["mx_b"].astype(np.int32) + rng.integers(-3, 4, extra["mx_b"].shape)).astype(np.uint8)
    bias = np.random.default_rng(42).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    out, name = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, bias=bias, ldc=ldc, **extra)
    assert name.startswith("skinnyx_mxfp4")
    want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[dtype_c], bias=bias)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()
    if dtype_c == "f32":
        tile, tname = run_gemm(a, b, M, N, K, "mxfp4", "f32", bias=bias, family=_capi.KERNEL_TILE,
                               **extra)
        assert not tname.startswith("skinny")
        assert G.rel_l2(out[:, :N], tile) <= 1e-5


@pytest.mark.parametrize("M,N,K", [(64, 14336, 4096), (17, 8, 4096), (33, 777, 8192), (48, 6000, 4096),
                                   (32, 1000, 8192)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_skinny_mxfp4_up_to_64_rows(gpu, M, N, K, dtype_c):
    a, b, extra = operands(M, N, K, "mxfp4", seed=45, b_std=0.05)
    rng = np.random.default_rng(46)
    extra["mx_a"] = (extra["mx_a"].astype(np.int32) + rng.integers(-3, 4, extra["mx_a"].shape)).astype(np.uint8)
    extra["mx_b"] = (extra["mx_b"].astype(np.int32) + rng.integers(-3, 4, extra["mx_b"].shape)).astype(np.uint8)
    bias = rng.standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, bias=bias, ldc=N + 8, **extra)
    assert name.startswith("skinnyx_mxfp4_m64")
    want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[dtype_c], bias=bias)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(16, 4096, 14336), (3, 8, 12288), (48, 777, 28672), (64, 4104, 16384),
                                   (16, 520, 11264), (40, 64, 4608), (1, 1000, 32768), (33, 136, 6144)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_skinny_mxfp4_long_rows(gpu, M, N, K, dtype_c):
    """MXFP4 rows that are not 2 or 4 KiB of nibbles: K ranges, the last one possibly short
    (a wave behind the row's end multiplies zeros under unit scales)."""
    a, b, extra = operands(M, N, K, "mxfp4", seed=77, b_std=0.05)
    rng = np.random.default_rng(80)   # spread the block scales: a wrong byte must not go unnoticed
    extra["mx_a"] = (extra["mx_a"].astype(np.int32) + rng.integers(-3, 4, extra["mx_a"].shape)).astype(np.uint8)
    extra["mx_b"] = (extra["mx_b"].astype(np.int32) + rng.integers(-3, 4, extra["mx_b"].shape)).astype(np.uint8)
    bias = np.random.default_rng(78).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, bias=bias, ldc=N + 8, **extra)
    assert name.startswith("skinnyx_mxfp4_m64")
    want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[dtype_c], bias=bias)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


def test_skinny_long_rows_keep_non_finite_inputs_in_their_row(gpu):
    """A NaN in one activation row reaches that output row only, also where the last K range is
    short and some waves multiply nothing."""
    M, N, K = 16, 256, 2304
    a, b, _ = operands(M, N, K, "bf16", seed=79, b_std=0.05)
    a = np.array(a, copy=True)
    a[0, 0] = 0x7FC0          # bf16 NaN in the first line of the activations
    out, name = run_gemm(a, b, M, N, K, "bf16", "f32", family=_capi.KERNEL_SKINNY)
    assert "_m64_" in name
    assert np.isnan(out[0]).all()
    assert np.isfinite(out[1:]).all()


@pytest.mark.parametrize("M,N,K", [(128, 4096, 14336), (96, 4096, 4096), (264, 520, 4096), (1000, 1000, 8192),
                                   (512, 4096, 4096), (72, 8, 4096), (128, 14336, 4096)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "bf16"), ("f16", "f32"), ("bf16", "f16")])
def test_split_k_on_few_output_tiles(gpu, M, N, K, dtype_ab, dtype_c):
    """At most 128 output tiles of 128 x 128 and long rows: AUTO cuts K into 4..16 ranges, one
    copy of the tile grid per range, fp32 planes in the library's workspace, summed in range
    order by a second kernel that applies bias and cast.  Edge tiles, a padded output pitch,
    and the same bits on a second run."""
    a, b, _ = operands(M, N, K, dtype_ab, seed=95, b_std=0.05)
    bias = np.random.default_rng(96).standard_normal(N).astype(np.float32)
    ldc = N + 8
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc)
    assert name.startswith("splitk_")
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
    check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()
    again, _ = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc)
    assert np.array_equal(out[:, :N].view(np.uint8), again[:, :N].view(np.uint8))
    # the unsplit kernels give the same result up to fp32 summation order
    if dtype_c == "f32":
        whole, wname = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, wg_tile=(64, 64))
        assert wname.startswith("tile")
        assert G.rel_l2(out[:, :N], whole) <= 1e-5


@pytest.mark.parametrize("M,N,K", [(128, 4096, 14336), (264, 520, 8192), (96, 1000, 16384), (512, 2048, 16384)])
@pytest.mark.parametrize("dtype_ab", ["fp8_e4m3", "mxfp4"])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_split_k_fp8_and_mxfp4(gpu, M, N, K, dtype_ab, dtype_c):
    """Split K on the fp8 and MXFP4 128 x 128 kernels: the tensor scales are applied after the
    planes are added; MXFP4 ranges start on whole 16-byte granules of the scale planes."""
    a, b, extra = operands(M, N, K, dtype_ab, seed=97, b_std=0.05)
    if dtype_ab == "mxfp4":
        rng = np.random.default_rng(98)
        extra["mx_a"] = (extra["mx_a"].astype(np.int32) + rng.integers(-3, 4, extra["mx_a"].shape)).astype(np.uint8)
        extra["mx_b"] = (extra["mx_b"].astype(np.int32) + rng.integers(-3, 4, extra["mx_b"].shape)).astype(np.uint8)
    bias = np.random.default_rng(99).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=N + 8, **extra)
    assert name.startswith("splitk_")
    if dtype_ab == "mxfp4":
        want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[dtype_c], bias=bias)
        bar = 1e-5
    else:
        want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
        bar = 1e-4
    check(out, want, dtype_c, N, bar=bar if dtype_c == "f32" else REL_L2_BAR)
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


def test_long_rows_above_32_activation_rows_take_split_k(gpu):
    """AUTO on rows the decode kernels cut into K ranges: M <= 32 stays with them, 32 < M <= 64
    goes to split K on the 128 x 128 kernel for rows of more than 32 KiB where the shape allows
    it (N % 8 == 0)."""
    for (M, N, K, dt, want) in ((32, 4096, 28672, "bf16", "skinnyx_bf16_m64"),
                                (48, 4096, 14336, "bf16", "skinnyx_bf16_m64"),
                                (48, 4096, 28672, "bf16", "splitk_bf16"),
                                (64, 4096, 20480, "f16", "splitk_f16"),
                                (64, 4100, 28672, "bf16", "skinnyx_bf16_m64"),
                                (64, 14336, 4096, "bf16", "skinnyx_bf16_m64"),
                                (64, 4096, 28672, "fp8_e4m3", "skinnyx_fp8_m64"),
                                (64, 4096, 40960, "fp8_e4m3", "splitk_fp8")):
        a, b, extra = operands(M, N, K, dt, seed=93, b_std=0.05)
        out, name = run_gemm(a, b, M, N, K, dt, "f32", **extra)
        assert name.startswith(want), (M, N, K, dt, name)
        if dt == "fp8_e4m3":
            ref = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=G.F32)
        else:
            ref = G.gemm(a, b, _DT[dt], G.F32)
        check(out, ref, "f32", N, bar=1e-4 if dt == "fp8_e4m3" else 1e-5)


def test_skinny_fp8_falls_back_to_tile_kernels(gpu):
    # rows shorter than 4 KiB or not whole 512-byte slices, or M > 64: AUTO keeps the tile family
    for (M, N, K) in ((16, 256, 1024), (65, 256, 4096), (17, 256, 11008)):
        a, b, extra = operands(M, N, K, "fp8_e4m3", seed=33)
        out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", **extra)
        assert name.startswith("tile")
        check(out, G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=G.F32), "f32", N,
              bar=1e-4)


@pytest.mark.parametrize("M,N,K", [(8, 8, 128), (264, 520, 128), (504, 1000, 192), (1000, 264, 1024),
                                   (2056, 1800, 256), (256, 776, 320), (256, 256, 136), (512, 264, 1016),
                                   (264, 256, 7008), (256, 512, 144), (256, 256, 240)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "bf16"), ("f16", "f32"), ("fp8_e4m3", "bf16"),
                                              ("fp8_e4m3", "f32")])
def test_stream_kernels_edge_tiles(gpu, M, N, K, dtype_ab, dtype_c):
    """M and N multiples of 8 but not of the 256 x 256 tile: row groups past the end re-read
    valid rows, the epilogue stores only what is inside, pad columns stay untouched.  K that
    does not end on a 128-byte step: the last 1..7 granules are multiplied after the loop."""
    if dtype_ab == "fp8_e4m3" and K % 16:
        pytest.skip("rows are whole 16-byte granules")
    a, b, extra = operands(M, N, K, dtype_ab, seed=51, b_std=0.05)
    bias = np.random.default_rng(52).standard_normal(N).astype(np.float32)
    ldc = N + 16
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc,
                         family=_capi.KERNEL_TILE, wg_tile=(256, 256), **extra)
    assert name.startswith("stream_")
    if dtype_ab == "fp8_e4m3":
        want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
    else:
        want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
    bar = REL_L2_BAR if dtype_c != "f32" else (1e-4 if dtype_ab == "fp8_e4m3" else 1e-5)
    if M * N >= 4096:
        check(out, want, dtype_c, N, bar=bar)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(256, 256, 1024), (264, 520, 1088), (384, 1000, 1152), (256, 384, 1216),
                                   (512, 264, 1408), (256, 256, 1472), (264, 256, 1536), (256, 512, 1600),
                                   (1000, 1024, 1664), (256, 256, 1728), (504, 776, 1800), (256, 128, 2120),
                                   (2048, 2048, 2048)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "bf16"), ("f16", "f32")])
def test_stream_128_with_nine_slot_ring(gpu, M, N, K, dtype_ab, dtype_c):
    """The 128 x 128 stream kernel with four K-steps requested ahead (nine LDS slots), which AUTO
    takes for at most one workgroup per CU and two or more tile rows.  K-step counts 16 (the
    minimum), 17, 18, 19 (one whole steady group of nine trips + prologue depth exactly), 22, 23,
    24, 25, 26, 27, 28 + a tail of granules, 33 + a tail, 32; edge tiles in M and N.  The same
    sums as the five-slot kernel (same K order, same accumulation)."""
    a, b, _ = operands(M, N, K, dtype_ab, seed=61, b_std=0.05)
    bias = np.random.default_rng(62).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, wg_tile=(128, 128),
                         family=_capi.KERNEL_TILE)
    assert name == f"stream_{dtype_ab}_128x128_w2x2_ring9_{dtype_c}"
    check(out, G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias), dtype_c, N,
          bar=REL_L2_BAR if dtype_c != "f32" else 1e-5)
    five, five_name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias,
                               variant=_variant_id(f"stream_{dtype_ab}_128x128_w2x2_{dtype_c}"))
    assert five_name == f"stream_{dtype_ab}_128x128_w2x2_{dtype_c}"
    assert np.array_equal(out, five)


def test_nine_slot_ring_is_left_to_grids_of_one_workgroup_per_cu(gpu):
    name = lambda *shape: AG.GemmPlan.create(*shape, "bf16", "bf16").info.name.decode()
    assert name(256, 14336, 4096) == "stream_bf16_128x128_w2x2_ring9_bf16"      # 224 tiles, two tile rows
    assert name(128, 28672, 4096) == "stream_bf16_128x128_w2x2_bf16"            # one tile row: HBM-bound
    assert name(512, 14336, 4096) == "stream_bf16_128x128_w2x2_bf16"            # 448 tiles: two per CU
    assert AG.GemmPlan.create(256, 14336, 4096, "bf16", "bf16").info.lds_bytes == 9 * 128 * 128


# ---- edge cases: ragged M / N, K tails, leading dimensions, epilogue -----------------

@pytest.mark.parametrize("M,N,K", [(1, 1, 8), (65, 16, 8), (130, 257, 72), (300, 520, 776), (129, 1, 64)])
@pytest.mark.parametrize("dtype_ab", ["bf16", "f16"])
def test_tile_ragged_shapes_and_k_tails(gpu, M, N, K, dtype_ab):
    a, b, _ = operands(M, N, K, dtype_ab, seed=3, b_std=0.1)
    out, name = run_gemm(a, b, M, N, K, dtype_ab, "f32", family=_capi.KERNEL_TILE)
    assert name.startswith("tile")
    check(out, G.gemm(a, b, _DT[dtype_ab], G.F32), "f32", N, bar=1e-5)


def test_tile_fp8_k_tail(gpu):
    M, N, K = 100, 200, 16 * 13
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=4, b_std=1.0)
    out, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", **ex)
    check(out, G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=G.F32), "f32", N, bar=1e-4)


def test_leading_dimensions(gpu):
    M, N, K, lda, ldb, ldc = 200, 136, 96, 128, 104, 160
    rng = np.random.default_rng(6)
    a = F.f32_to_bf16_bits(rng.standard_normal((M, lda)).astype(np.float32))
    b = F.f32_to_bf16_bits((rng.standard_normal((N, ldb)) * 0.1).astype(np.float32))
    out, _ = run_gemm(a, b, M, N, K, "bf16", "bf16", lda=lda, ldb=ldb, ldc=ldc,
                      family=_capi.KERNEL_TILE)
    check(out, G.gemm(a[:, :K], b[:, :K], G.BF16, G.BF16), "bf16", N)
    assert np.all(out[:, N:] == 0x7FC1)  # padding columns of C are not written


@pytest.mark.parametrize("ldc", [0, 203])
def test_bias_scale_and_output_types(gpu, ldc):
    M, N, K = 140, 200, 128
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=8, b_std=1.0)
    bias = np.random.default_rng(10).standard_normal(N).astype(np.float32)
    for dtype_c in ("f32", "bf16", "f16"):
        out, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias, ldc=ldc, **ex)
        want = G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
        check(out, want, dtype_c, N)


# ---- known answers of the reference's MFMA tests ---------------------------------------

@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "kat.json")) as f:
        return {c["name"]: c for c in json.load(f)["cases"]}


def test_kat_bf16_all_ones(gpu, kat):
    c = kat["bf16_16x16x32_all_ones"]
    a = np.full((16, 32), int(c["a_bits"], 16), np.uint16)
    out, _ = run_gemm(a, a, 16, 16, 32, "bf16", "f32", family=_capi.KERNEL_TILE)
    assert np.all(out == c["expected"])
    out, _ = run_gemm(a, a, 16, 16, 32, "bf16", "f32", family=_capi.KERNEL_SKINNY)
    assert np.all(out == c["expected"])


def test_kat_fp8_scaled(gpu, kat):
    c = kat["fp8_scaled_nonidentity"]
    a = np.full((16, 128), int(c["a_byte"], 16), np.uint8)
    b = np.full((16, 128), int(c["b_byte"], 16), np.uint8)
    out, _ = run_gemm(a, b, 16, 16, 128, "fp8_e4m3", "f32", scale_a=c["scale_a"], scale_b=c["scale_b"])
    assert np.all(out == c["expected"])


def test_kat_fp8_split_k_accumulate(gpu, kat):
    c = kat["fp8_split_k_accum"]
    a = np.empty((16, 128), np.uint8)
    b = np.empty((16, 128), np.uint8)
    a[:, :64], a[:, 64:] = (int(v, 16) for v in c["a_bytes_halves"])
    b[:, :64], b[:, 64:] = (int(v, 16) for v in c["b_bytes_halves"])
    out, _ = run_gemm(a, b, 16, 16, 128, "fp8_e4m3", "f32", scale_a=1.0, scale_b=1.0,
                      bias=np.full(16, c["c_init"], np.float32))
    assert np.all(out == c["expected"])


def test_kat_mxfp4_block_scales(gpu):
    # e2m1 code 2 = 1.0, code 3 = 1.5; e8m0 0x81 = 4, 0x80 = 2: 256 * 1.0 * 1.5 * 8 = 3072
    a = np.full((16, 128), 0x22, np.uint8)
    b = np.full((16, 128), 0x33, np.uint8)
    out, _ = run_gemm(a, b, 16, 16, 256, "mxfp4", "f32", mx_a=np.full((16, 8), 0x81, np.uint8),
                      mx_b=np.full((16, 8), 0x80, np.uint8))
    assert np.all(out == 3072.0)


# ---- full-size properties (configuration 2: bf16 8192^3) -------------------------------

@pytest.fixture(scope="module")
def big():
    M = N = K = 8192
    a, b, _ = operands(M, N, K, "bf16")
    return M, N, K, a, b


def test_config2_full_size_row_sample_determinism_and_scaling(gpu, big):
    M, N, K, a, b = big
    out, name = run_gemm(a, b, M, N, K, "bf16", "bf16")
    assert "256x256" in name
    rows = np.random.default_rng(0).choice(M, 48, replace=False)
    rows = np.concatenate([rows, [0, 255, 256, M - 1]])
    want = G.gemm(a[rows], b, G.BF16, G.BF16)
    check(out[rows], want, "bf16", N)
    cols = np.random.default_rng(1).choice(N, 32, replace=False)
    want_c = G.gemm(a, b[cols], G.BF16, G.BF16)
    check(out[:, cols], want_c, "bf16", 32)
    # run-to-run determinism
    out2, _ = run_gemm(a, b, M, N, K, "bf16", "bf16")
    assert np.array_equal(out, out2)
    # scaling A by 4 is exact in bf16 and in the fp32 accumulator
    a4 = F.f32_to_bf16_bits(F.bf16_bits_to_f32(a) * 4.0)
    out4, _ = run_gemm(a4, b, M, N, K, "bf16", "bf16")
    assert np.array_equal(F.bf16_bits_to_f32(out4), F.bf16_bits_to_f32(out) * 4.0)


def _sampled_rows_and_cols(M, N):
    rows = np.random.default_rng(0).choice(M, 48, replace=False)
    rows = np.concatenate([rows, [0, 255, 256, M - 1]])
    cols = np.random.default_rng(1).choice(N, 32, replace=False)
    return rows, cols


def test_config3_full_size_fp8_row_sample_determinism_and_scaling(gpu):
    # configuration 3 at the size the bench times: 8192^3, operands e4m3 of N(0,1) sources with
    # s = absmax / 448 (seeds 42 / 43), bf16 output with the scales applied in the epilogue
    M = N = K = 8192
    a, b, ex = operands(M, N, K, "fp8_e4m3", a_std=1.0, b_std=1.0)
    out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", "bf16", **ex)
    assert name == "stream_fp8_256x256_w2x4_walk_bf16"   # 1024 tiles: four per workgroup
    rows, cols = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm_fp8(a[rows], b, ex["scale_a"], ex["scale_b"], out_dtype=G.BF16), "bf16", N)
    check(out[:, cols], G.gemm_fp8(a, b[cols], ex["scale_a"], ex["scale_b"], out_dtype=G.BF16),
          "bf16", len(cols))
    # against the float64-accumulated product on the sampled rows: at most 2 bf16 ulp
    w64 = G.gemm_fp8(a[rows], b, ex["scale_a"], ex["scale_b"], out_dtype=G.BF16, accumulate="f64")
    w64f = F.bf16_bits_to_f32(w64)
    solid = np.abs(w64f) > 1e-2 * np.sqrt(np.mean(w64f.astype(np.float64) ** 2))
    ulp = np.abs(out[rows].astype(np.int32) - w64.astype(np.int32))
    assert ulp[solid].max() <= 2 and np.mean(ulp[solid] > 1) < 1e-3
    # run-to-run determinism
    out2, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", "bf16", **ex)
    assert np.array_equal(out, out2)
    # a tensor scale four times as large is exact in the fp32 epilogue and in bf16
    out4, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", "bf16", scale_a=np.float32(ex["scale_a"]) * 4,
                       scale_b=ex["scale_b"])
    assert np.array_equal(F.bf16_bits_to_f32(out4), F.bf16_bits_to_f32(out) * 4.0)


def test_config5_full_size_mxfp4_row_sample_determinism_and_scaling(gpu):
    # configuration 5 at the size the bench times: 4096 x 14336 x 4096, both operands MXFP4 from
    # N(0,1) sources (seeds 42 / 43), e8m0 from the absmax of every 32-wide K block
    M, N, K = 4096, 14336, 4096
    a, b, ex = operands(M, N, K, "mxfp4", a_std=1.0, b_std=1.0)
    out, name = run_gemm(a, b, M, N, K, "mxfp4", "bf16", **ex)
    assert name.startswith("stream_mxfp4_")
    rows, cols = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm_mxfp4(a[rows], ex["mx_a"][rows], b, ex["mx_b"], out_dtype=G.BF16),
          "bf16", N)
    check(out[:, cols], G.gemm_mxfp4(a, ex["mx_a"], b[cols], ex["mx_b"][cols], out_dtype=G.BF16),
          "bf16", len(cols))
    out32, _ = run_gemm(a[:512], b, 512, N, K, "mxfp4", "f32", mx_a=ex["mx_a"][:512], mx_b=ex["mx_b"])
    check(out32, G.gemm_mxfp4(a[:512], ex["mx_a"][:512], b, ex["mx_b"], out_dtype=G.F32), "f32", N,
          bar=1e-5)
    # run-to-run determinism
    out2, _ = run_gemm(a, b, M, N, K, "mxfp4", "bf16", **ex)
    assert np.array_equal(out, out2)
    # every e8m0 byte of A one higher doubles every product exactly
    assert ex["mx_a"].max() < 254
    outx2, _ = run_gemm(a, b, M, N, K, "mxfp4", "bf16", mx_a=ex["mx_a"] + np.uint8(1), mx_b=ex["mx_b"])
    assert np.array_equal(F.bf16_bits_to_f32(outx2), F.bf16_bits_to_f32(out) * 2.0)


def _variant_id(name):
    lib = _capi.load()
    cfg, info = _capi.Config(), _capi.KernelInfo()
    cfg.M = cfg.N = cfg.K = 512
    for i in range(lib.astergemm_variant_count()):
        _capi.check(lib.astergemm_variant_info(i, ctypes.byref(cfg), ctypes.byref(info)))
        if info.name.decode() == name:
            return info.variant
    raise KeyError(name)


@pytest.mark.parametrize("M,N", [(512, 32768 + 520), (33288, 512), (1024, 16384 + 264)])
@pytest.mark.parametrize("dtype_ab,dtype_c,K", [("bf16", "bf16", 264), ("f16", "f32", 128),
                                                ("fp8_e4m3", "bf16", 384), ("mxfp4", "bf16", 512)])
def test_whole_rounds_plus_tail_split(gpu, M, N, dtype_ab, dtype_c, K):
    # 256 x 256 tiles that do not fill whole rounds of the 256 CUs: the columns (rows) that do go
    # to the 256 x 256 kernel, the rest to the 128 x 128 kernel; bias and scales follow the cut
    a, b, ex = operands(M, N, K, dtype_ab, a_std=1.0, b_std=1.0 if dtype_ab != "bf16" else 0.02)
    bias = np.random.default_rng(3).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, wg_tile=(256, 256), **ex)
    assert "tail128" in name, name
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias, **ex)
    check(out, want, dtype_c, N)
    # the same bits as the two kernels give when each runs the whole problem
    plain = name.replace("_tail128", "")
    waves = plain.split("_")[3]
    for vname, rows, cols in ((plain, slice(0, 256), slice(0, 256)),
                              (plain.replace("256x256_" + waves, "128x128_w2x2"),
                               slice(M - 128, M), slice(N - 128, N))):
        whole, wname = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias,
                                variant=_variant_id(vname), **ex)
        assert wname == vname
        assert np.array_equal(out[rows, cols], whole[rows, cols])


def test_identity_operand_is_exact_at_full_width(gpu):
    # B = I: every output is one product plus zeros, so C == A bit for bit.
    M, N = 512, 8192
    a = F.f32_to_bf16_bits(np.random.default_rng(2).standard_normal((M, N)).astype(np.float32))
    eye = np.zeros((N, N), np.uint16)
    eye[np.arange(N), np.arange(N)] = 0x3F80
    out, _ = run_gemm(a, eye, M, N, N, "bf16", "bf16", family=_capi.KERNEL_TILE)
    assert np.array_equal(out, a)


@pytest.mark.parametrize("dtype_ab,M", [("bf16", 2048), ("fp8_e4m3", 2048), ("fp8_e4m3", 4096),
                                        ("mxfp4", 4096)])
def test_band_tile_order_writes_every_tile_once(gpu, dtype_ab, M):
    # B = I at a size whose tile grid divides by 8 x 32 (all XCDs on one band of eight tile
    # rows; with 4096 rows there are more tiles than CUs and the tile walks run): each output
    # is one product plus zeros, so C is A's values bit for bit and a tile that is skipped,
    # written twice from the wrong place or swapped with another shows
    N = K = 8192
    rng = np.random.default_rng(11)
    x = rng.standard_normal((M, K)).astype(np.float32)
    ex = {}
    if dtype_ab == "bf16":
        a = F.f32_to_bf16_bits(x)
        b = np.zeros((N, K), np.uint16)
        b[np.arange(N), np.arange(N)] = 0x3F80
        want = a
    elif dtype_ab == "fp8_e4m3":
        a = F.e4m3_encode(x)
        b = np.zeros((N, K), np.uint8)
        b[np.arange(N), np.arange(N)] = F.e4m3_encode_scalar(1.0)
        ex = dict(scale_a=np.float32(1), scale_b=np.float32(1))
        want = F.f32_to_bf16_bits(F.e4m3_decode(a))
    else:
        a, mxa = F.quantize_mxfp4(x)
        codes = np.zeros((N, K), np.uint8)
        codes[np.arange(N), np.arange(N)] = F.e2m1_encode(np.ones(1, np.float32))[0]
        b = F.pack_nibbles(codes)
        ex = dict(mx_a=mxa, mx_b=np.full((N, K // 32), 127, np.uint8))
        want = F.f32_to_bf16_bits(F.dequantize_mxfp4(a, mxa))
    out, name = run_gemm(a, b, M, N, K, dtype_ab, "bf16", **ex)
    assert name.startswith("stream_") and "256x256" in name, name
    assert ("_walk_" in name) == (M == 4096), name
    # as values: a negative zero of A comes out as the accumulator's positive zero
    assert np.array_equal(F.bf16_bits_to_f32(out), F.bf16_bits_to_f32(want))


# ---- every pre-built tile variant, selected by its id ---------------------------------------

def _tile_variants():
    import ctypes
    lib = _capi.load()
    c = _capi.Config()
    c.M = c.N = 512
    c.K = 1024
    out = []
    for i in range(lib.astergemm_variant_count()):
        info = _capi.KernelInfo()
        _capi.check(lib.astergemm_variant_info(i, ctypes.byref(c), ctypes.byref(info)))
        name = info.name.decode()
        if info.family != _capi.KERNEL_TILE:
            continue
        kind, ab = name.split("_")[0], name.split("_")[1]
        out.append((i + 1, name, {"fp8": "fp8_e4m3"}.get(ab, ab), name.rsplit("_", 1)[1]))
    return out


@pytest.mark.parametrize("vid,name,dtype_ab,dtype_c", _tile_variants(), ids=lambda v: str(v))
def test_every_tile_variant(gpu, vid, name, dtype_ab, dtype_c):
    M, N, K = 512, 768, 1536  # whole 256-tiles; 24 / 12 / 6 K-steps of 128 bytes (16-bit / fp8 / fp4)
    if name.startswith("splitk"):
        K = {"fp8_e4m3": 8192, "mxfp4": 8192}.get(dtype_ab, 4096)  # 64 (MXFP4: 32) steps of 128 bytes
    if "tail128" in name:
        M, N, K = 512, 32768 + 256, 512  # 2 x 129 tiles of 256 x 256: one whole round and a rest
    if "_walk_" in name:
        M, N, K = 512, 32768 + 256, 1024  # 258 tiles: more than one per workgroup, four K-steps
    a, b, ex = operands(M, N, K, dtype_ab, seed=11, a_std=1.0, b_std=1.0 if dtype_ab != "bf16" else 0.05)
    bias = np.random.default_rng(12).standard_normal(N).astype(np.float32)
    path, b_dev, ex_dev = "lds", b, ex
    mxl = "rows"
    if name.startswith("streamdb_mxfp4"):  # payload in step order, scale plane in lane order
        from aster_amd.kittens_helpers import (shuffle_scales_e8m0_lanes, shuffle_scales_e8m0_lanes128,
                                               shuffle_weight_bytes)
        path, b_dev = "direct_b_k8", shuffle_weight_bytes(b)
        ex_dev = dict(ex, mx_b=shuffle_scales_e8m0_lanes(ex["mx_b"]))
        if "_sal_" in name:    # and A's plane in lane order as well
            mxl, ex_dev["mx_a"] = "lanes128", shuffle_scales_e8m0_lanes128(ex["mx_a"])
    elif name.startswith("streamdb_fp8"):  # byte rows in step order
        from aster_amd.kittens_helpers import shuffle_weight_bytes
        path, b_dev = "direct_b_k8", shuffle_weight_bytes(b)
    elif name.startswith("streamdb"):  # B pre-shuffled in K8 order
        from aster_amd.kittens_helpers import shuffle_weight_k8
        path, b_dev = "direct_b_k8", shuffle_weight_k8(np.ascontiguousarray(b).view(np.uint16))
    a_dev = a
    if name.startswith("directab"):  # A and B both in the reference's shuffle_weight order
        from aster_amd.kittens_helpers import shuffle_weight
        path = "direct_ab"
        a_dev = shuffle_weight(np.ascontiguousarray(a).view(np.uint16))
        b_dev = shuffle_weight(np.ascontiguousarray(b).view(np.uint16))
    plan = AG.GemmPlan.create(M, N, K, dtype_ab, dtype_c, has_bias=True, variant=vid, operand_path=path,
                              mx_a_layout=mxl)
    assert plan.info.name.decode() == name
    out = np.zeros((M, N), dtype=_OUT_NP[dtype_c])
    bufs = {}
    for key, arr in dict(a=a_dev, b=b_dev, c=out, bias=bias, **{k: np.asarray(v) for k, v in ex_dev.items()}).items():
        arr = np.ascontiguousarray(arr if arr.ndim else arr.reshape(1).astype(np.float32))
        bufs[key] = GpuBuffer(arr.nbytes)
        bufs[key].copy_from_host(arr)
    kw = {k: bufs[k].ptr_value for k in ("scale_a", "scale_b", "mx_a", "mx_b") if k in bufs}
    print(f"launch {name}", flush=True)
    plan.run(bufs["a"].ptr_value, bufs["b"].ptr_value, bufs["c"].ptr_value, bias=bufs["bias"].ptr_value, **kw)
    bufs["c"].copy_to_host(out)
    for bf in bufs.values():
        bf.free()
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias, **ex)
    check(out, want, dtype_c, N, bar=1e-3 if dtype_c != "f32" else 1e-4)


def test_stream_kernel_is_the_default_for_whole_tiles(gpu):
    p = AG.GemmPlan.create(8192, 8192, 8192, "bf16", "bf16")
    assert p.info.name.decode().startswith("stream_bf16_256x256")
    assert p.info.lds_bytes == 163840
    # edge tiles in units of 8 rows and a K tail of whole granules are its own
    assert AG.GemmPlan.create(8192, 8192, 8200, "bf16", "bf16").info.name.decode().startswith("stream_")
    assert AG.GemmPlan.create(8000, 8104, 8192, "bf16", "bf16").info.name.decode().startswith("stream_")
    # shapes it does not take fall back to the general tile kernel
    assert AG.GemmPlan.create(8192, 8100, 8192, "bf16", "bf16").info.name.decode().startswith("tile_")
    with pytest.raises(_capi.AsterGemmError, match="16-byte granules"):
        AG.GemmPlan.create(8192, 8192, 8196, "bf16", "bf16", lda=8200, ldb=8200)


@pytest.mark.parametrize("K", [64, 128, 192, 256, 320, 384, 448, 512, 576, 640, 704])
def test_stream_kernel_every_ring_phase(gpu, K):
    # K-steps 1..11: prologue only, partial rings, steady trips + every tail length
    a, b, _ = operands(256, 512, K, "bf16", seed=13, b_std=0.1)
    out, name = run_gemm(a, b, 256, 512, K, "bf16", "f32", family=_capi.KERNEL_TILE, wg_tile=(256, 256))
    assert name.startswith("stream")
    check(out, G.gemm(a, b, G.BF16, G.F32), "f32", 512, bar=1e-5)


@pytest.mark.parametrize("ksteps", list(range(1, 14)))
def test_fp8_stream_kernel_128_every_ring_phase(gpu, ksteps):
    M, N, K = 128, 256, 128 * ksteps
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=19, b_std=1.0)
    out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", family=_capi.KERNEL_TILE,
                         wg_tile=(128, 128), **ex)
    assert name.startswith("stream_fp8_128")
    check(out, G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=G.F32), "f32", N, bar=1e-4)


@pytest.mark.parametrize("ksteps", list(range(1, 16)) + [20, 21])
def test_fp8_stream_kernel_every_ring_phase(gpu, ksteps):
    # 128-byte K-steps 1..15, 20, 21: prologue only, every tail length of the six-trip slot
    # period, one and two steady periods followed by every kind of tail
    M, N, K = 256, 512, 128 * ksteps
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=17, b_std=1.0)
    out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", family=_capi.KERNEL_TILE,
                         wg_tile=(256, 256), **ex)
    assert name.startswith("stream_fp8")
    check(out, G.gemm(a, b, G.FP8_E4M3, G.F32, **ex), "f32", N, bar=1e-4)


def test_fp8_stream_and_tile_kernels_pair_granules_consistently(gpu):
    # the stream kernel visits the 128 K positions of a step in a different order than the
    # general tile kernel; both must agree with the oracle on data where a wrong pairing of
    # granules between A and B cannot cancel (distinct magnitude per 16-byte granule)
    M, N, K = 256, 256, 512
    rng = np.random.default_rng(23)
    gran = 2.0 ** rng.integers(-3, 4, size=(K // 16)).astype(np.float32)
    xa = (rng.standard_normal((M, K)).astype(np.float32)) * np.repeat(gran, 16)[None, :]
    xb = rng.standard_normal((N, K)).astype(np.float32)
    a, sa = F.quantize_fp8_tensor(xa)
    b, sb = F.quantize_fp8_tensor(xb)
    want = G.gemm(a, b, G.FP8_E4M3, G.F32, scale_a=sa, scale_b=sb)
    for tile, prefix in ((256, "stream_fp8_256"), (128, "stream_fp8_128"), (64, "tile_fp8")):
        out, name = run_gemm(a, b, M, N, K, "fp8_e4m3", "f32", scale_a=sa, scale_b=sb,
                             family=_capi.KERNEL_TILE, wg_tile=(tile, tile))
        assert name.startswith(prefix)
        check(out, want, "f32", N, bar=1e-4)


def test_bench_rotate_uses_every_operand_set(gpu):
    # three weight matrices and three outputs in turn: afterwards every output holds the
    # product with its own weights, and the total time is positive
    M, N, K = 16, 512, 2048
    a, _, _ = operands(M, N, K, "bf16", seed=31)
    plan = AG.GemmPlan.create(M, N, K, "bf16", "f32")
    bufs, sets, weights = [], [], []
    da = GpuBuffer(a.nbytes)
    da.copy_from_host(a)
    for i in range(3):
        _, b, _ = operands(M, N, K, "bf16", seed=40 + i, b_std=0.05)
        weights.append(b)
        db, dc = GpuBuffer(b.nbytes), GpuBuffer(M * N * 4)
        db.copy_from_host(b)
        bufs += [db, dc]
        sets.append({"dA": da.ptr_value, "dB": db.ptr_value, "dC": dc.ptr_value})
    total = plan.bench_rotate(sets, 7)
    assert total > 0
    for i in range(3):
        out = np.zeros((M, N), np.float32)
        bufs[2 * i + 1].copy_to_host(out)
        check(out, G.gemm(a, weights[i], G.BF16, G.F32), "f32", N, bar=1e-5)
    for bf in bufs + [da]:
        bf.free()
    with pytest.raises(_capi.AsterGemmError):
        plan.bench_rotate([], 3)


@pytest.mark.parametrize("M,N,K", [(16, 512, 2048), (16, 520, 14336), (128, 4096, 14336)])
def test_bench_graph_replays_the_captured_launches(gpu, M, N, K):
    """Launches captured once into a HIP graph and replayed (a decode kernel, one in K ranges with
    the library's partial-sum workspace, split K with its second kernel): every operand set ends
    up with the product of its own weights, three replays after the untimed one, and the outputs
    are the bits of eager launches."""
    a, _, _ = operands(M, N, K, "bf16", seed=31)
    plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16")
    bufs, sets, eager = [], [], []
    da = GpuBuffer(a.nbytes)
    da.copy_from_host(a)
    for i in range(3):
        _, b, _ = operands(M, N, K, "bf16", seed=40 + i, b_std=0.05)
        db, dc = GpuBuffer(b.nbytes), GpuBuffer(M * N * 2)
        db.copy_from_host(b)
        plan.run(da.ptr_value, db.ptr_value, dc.ptr_value)
        ref = np.zeros((M, N), np.uint16)
        dc.copy_to_host(ref)
        eager.append(ref)
        dc.copy_from_host(np.full((M, N), 0x7FC1, np.uint16))
        bufs += [db, dc]
        sets.append({"dA": da.ptr_value, "dB": db.ptr_value, "dC": dc.ptr_value})
    print(f"graph of 6 launches of {plan.info.name.decode()} M={M} N={N} K={K}", flush=True)
    total = plan.bench_graph(sets, 6, 3)
    assert total > 0
    for i in range(3):
        out = np.zeros((M, N), np.uint16)
        bufs[2 * i + 1].copy_to_host(out)
        assert np.array_equal(out, eager[i])
    for bf in bufs + [da]:
        bf.free()
    with pytest.raises(_capi.AsterGemmError):
        plan.bench_graph([], 3, 1)


@pytest.mark.parametrize("ksteps", [2, 4, 6, 8, 10, 12, 14])
@pytest.mark.parametrize("tile", [256, 128])
def test_mxfp4_stream_kernel_every_loop_phase(gpu, ksteps, tile):
    # 256-element K-steps in pairs (scales travel two K-steps at a time): final parts only,
    # the block before them, and one to five steady iterations; random nibbles and random
    # per-block scales, so a wrong block <-> scale byte pairing cannot cancel
    M, N, K = 256, 512, 256 * ksteps
    rng = np.random.default_rng(29 + ksteps)
    a = rng.integers(0, 256, (M, K // 2)).astype(np.uint8)
    b = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    mxa = rng.integers(118, 134, (M, K // 32)).astype(np.uint8)
    mxb = rng.integers(118, 134, (N, K // 32)).astype(np.uint8)
    out, name = run_gemm(a, b, M, N, K, "mxfp4", "f32", mx_a=mxa, mx_b=mxb,
                         family=_capi.KERNEL_TILE, wg_tile=(tile, tile))
    assert name.startswith(f"stream_mxfp4_{tile}")
    check(out, G.gemm_mxfp4(a, mxa, b, mxb, out_dtype=G.F32), "f32", N, bar=1e-5)


@pytest.mark.parametrize("ksteps", [2, 4, 6, 8, 10, 12, 14])
@pytest.mark.parametrize("dtype_c", ["f32", "bf16"])
def test_mxfp4_stream_kernel_eight_waves_every_loop_phase(gpu, ksteps, dtype_c):
    # the 256 x 256 kernel with 2 x 4 waves (wave tile 128 x 64): same loop phases, an edge tile
    # in M and N, random nibbles and per-block scales
    M, N, K = 264, 520, 256 * ksteps
    rng = np.random.default_rng(61 + ksteps)
    a = rng.integers(0, 256, (M, K // 2)).astype(np.uint8)
    b = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    mxa = rng.integers(118, 134, (M, K // 32)).astype(np.uint8)
    mxb = rng.integers(118, 134, (N, K // 32)).astype(np.uint8)
    out, name = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, mx_a=mxa, mx_b=mxb,
                         variant=_variant_id(f"stream_mxfp4_256x256_w2x4_{dtype_c}"))
    assert name == f"stream_mxfp4_256x256_w2x4_{dtype_c}"
    want = G.gemm_mxfp4(a, mxa, b, mxb, out_dtype=_DT[dtype_c])
    check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)


@pytest.mark.parametrize("K", [1024, 2048, 3072])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_mxfp4_tile_walk_equals_the_plain_kernel(gpu, K, dtype_c):
    """The tile walk (one workgroup per CU takes several tiles as one long K loop, the next tile's
    first K-steps arriving during the last trips of the current one) on more tiles than any
    device has CUs: the same bits as the one-tile-per-workgroup kernel, and sampled rows against
    the oracle.  The walk takes whole tiles only."""
    M, N = 4352, 4608   # 17 x 18 = 306 tiles of 256 x 256
    rng = np.random.default_rng(7 + K)
    a = rng.integers(0, 256, (M, K // 2)).astype(np.uint8)
    b = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    mxa = rng.integers(118, 134, (M, K // 32)).astype(np.uint8)
    mxb = rng.integers(118, 134, (N, K // 32)).astype(np.uint8)
    bias = rng.standard_normal(N).astype(np.float32)
    plain, pname = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, mx_a=mxa, mx_b=mxb, bias=bias,
                            variant=_variant_id(f"stream_mxfp4_256x256_w2x4_{dtype_c}"))
    walk, wname = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, mx_a=mxa, mx_b=mxb, bias=bias,
                           variant=_variant_id(f"stream_mxfp4_256x256_w2x4_walk_{dtype_c}"))
    assert pname == f"stream_mxfp4_256x256_w2x4_{dtype_c}" and wname == f"stream_mxfp4_256x256_w2x4_walk_{dtype_c}"
    assert np.array_equal(walk.view(np.uint8), plain.view(np.uint8))
    rows = np.unique(np.concatenate([rng.integers(0, M, 12), [0, 255, 256, M - 1]]))
    want = G.gemm_mxfp4(a[rows], mxa[rows], b, mxb, out_dtype=_DT[dtype_c], bias=bias)
    check(walk[rows], want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)


@pytest.mark.parametrize("K", [512, 640, 768, 896, 2048])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
def test_fp8_tile_walk_equals_the_plain_kernel(gpu, K, dtype_c):
    """The fp8 tile walk (one workgroup per CU takes several tiles in one launch; the next tile's
    first two K-steps arrive during the epilogue, whose stores stay in flight into the next tile)
    on more tiles than any device has CUs, K-step counts 4, 5, 6, 7 (every phase of the three A
    and two B slots at the end of a tile) and 16: the same bits as the one-tile-per-workgroup
    kernel, and sampled rows against the oracle.  The walk takes whole tiles only."""
    M, N = 4352, 4608   # 17 x 18 = 306 tiles of 256 x 256
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=5 + K, a_std=1.0, b_std=1.0)
    bias = np.random.default_rng(K).standard_normal(N).astype(np.float32)
    plain, pname = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias,
                            variant=_variant_id(f"stream_fp8_256x256_w2x4_{dtype_c}"), **ex)
    walk, wname = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias,
                           variant=_variant_id(f"stream_fp8_256x256_w2x4_walk_{dtype_c}"), **ex)
    assert pname == f"stream_fp8_256x256_w2x4_{dtype_c}" and wname == f"stream_fp8_256x256_w2x4_walk_{dtype_c}"
    assert np.array_equal(walk.view(np.uint8), plain.view(np.uint8))
    rows = np.unique(np.concatenate([np.random.default_rng(1).integers(0, M, 12), [0, 255, 256, M - 1]]))
    want = G.gemm_fp8(a[rows], b, ex["scale_a"], ex["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
    check(walk[rows], want, dtype_c, N)


def test_mxfp4_stream_kernel_falls_back_for_odd_kstep_counts(gpu):
    assert AG.GemmPlan.create(512, 512, 768, "mxfp4", "bf16", wg_tile=(256, 256)).info.name.decode() \
        .startswith("tile_mxfp4")
    assert AG.GemmPlan.create(4096, 14336, 4096, "mxfp4", "bf16").info.name.decode() \
        .startswith("stream_mxfp4")


@pytest.mark.parametrize("M,N,K", [(16, 14336, 4096), (1, 16, 2048), (5, 784, 8192), (13, 6000, 2048),
                                   (16, 48, 4096), (9, 4112, 8192), (16, 4096 + 16 * 7, 4096)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "f32"), ("f16", "f16"), ("bf16", "bf16")])
def test_skinny_direct_b_preshuffled_weights(gpu, M, N, K, dtype_ab, dtype_c):
    """operand_path = direct_b: B is handed over in the order of the reference's
    shuffle_weight (kittens_helpers.py:90-119); the result must equal the GEMM on the
    unshuffled weights.  Row ranges that start or end inside a 16-row chunk, single-workgroup
    grids, bias and a padded output pitch."""
    from aster_amd.kittens_helpers import shuffle_weight
    a, b, _ = operands(M, N, K, dtype_ab, seed=51, b_std=0.05)
    bias = np.random.default_rng(52).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    out, name = run_gemm(a, shuffle_weight(b), M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc,
                         operand_path="direct_b")
    assert name.startswith("skinnyd")
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
    check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N", [(16, 14336), (1, 16), (5, 784), (13, 6000), (16, 48), (9, 4112),
                                 (16, 4096 + 16 * 7)])
@pytest.mark.parametrize("dtype_ab,K,dtype_c", [("fp8_e4m3", 4096, "bf16"), ("fp8_e4m3", 2048, "f32"),
                                                ("fp8_e4m3", 8192, "f16"), ("mxfp4", 8192, "bf16"),
                                                ("mxfp4", 4096, "f32"), ("mxfp4", 16384, "f32")])
def test_skinny_direct_b_preshuffled_fp8_and_mxfp4_weights(gpu, M, N, dtype_ab, K, dtype_c):
    """operand_path = direct_b for the one-byte and nibble types: the payload rows in the step
    order of `shuffle_weight_bytes`, the MXFP4 scale plane in the order of `shuffle_scales_e8m0`;
    the result must equal the oracle's GEMM on the unshuffled weights, and the kernel that reads
    the same weights row-major through LDS to summation order.  Row ranges that start or end
    inside a 16-row block, single-workgroup grids, bias and a padded output pitch."""
    from aster_amd.kittens_helpers import shuffle_scales_e8m0, shuffle_weight_bytes
    a, b, ex = operands(M, N, K, dtype_ab, seed=57, b_std=0.05)
    bias = np.random.default_rng(58).standard_normal(N).astype(np.float32)
    ldc = (N + 11) & ~3
    ex_dev = dict(ex)
    if dtype_ab == "mxfp4":
        ex_dev["mx_b"] = shuffle_scales_e8m0(ex["mx_b"])
    out, name = run_gemm(a, shuffle_weight_bytes(np.asarray(b).view(np.uint8)), M, N, K, dtype_ab, dtype_c,
                         bias=bias, ldc=ldc, operand_path="direct_b", **ex_dev)
    assert name.startswith("skinnyd_" + ("fp8" if dtype_ab == "fp8_e4m3" else "mxfp4"))
    want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias, **ex)
    if dtype_c == "f32" or M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-4 if dtype_c == "f32" else REL_L2_BAR)
    else:  # few outputs: bound every element (see test_skinny_fp8_resident_activations)
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()
    plain, pname = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=ldc, **ex)
    assert not pname.startswith("skinnyd")
    assert G.rel_l2(G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(plain[:, :N], _DT[dtype_c])) \
        <= (1e-5 if dtype_c == "f32" else REL_L2_BAR)


# ---- B pre-shuffled in K8 order, loaded straight into MFMA operands (256 x 256 stream kernel) ---

@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (256, 256, 128), (512, 768, 576), (512, 512, 640),
                                   (264, 528, 704), (1000, 1008, 896), (256, 512, 960),
                                   (512, 256, 1280), (768, 1024, 1472), (2048, 2048, 4096)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "bf16"), ("f16", "f32")])
@pytest.mark.parametrize("tile_m", [256, 128])
def test_stream_direct_b_k8(gpu, M, N, K, dtype_ab, dtype_c, tile_m):
    # K steps of 64 elements: 1, 2, 9 (no steady group), 10 (one steady group exactly), 11, 14, 15,
    # 20, 23, 64; edge tiles in M (multiple of 8) and N (multiple of 16).  tile_m 128 is the
    # reference's own best mapping: 128 x 256 tiles, four waves side by side
    from aster_amd.kittens_helpers import shuffle_weight_k8
    a, b, _ = operands(M, N, K, dtype_ab)
    bias = np.random.default_rng(4).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, shuffle_weight_k8(b), M, N, K, dtype_ab, dtype_c, bias=bias,
                         operand_path="direct_b_k8", wg_tile=(tile_m, 256))
    assert name.startswith(f"streamdb_{dtype_ab}_{tile_m}x256_w{tile_m // 128}x4_")
    check(out, G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias), dtype_c, N)
    # the same K order on both operands as the LDS kernel: same products, same sums
    lds_out, lds_name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, wg_tile=(256, 256),
                                 family=_capi.KERNEL_TILE)
    if lds_name.startswith("stream_"):
        assert G.rel_l2(G.output_to_f32(out, _DT[dtype_c]), G.output_to_f32(lds_out, _DT[dtype_c])) <= 1e-5


@pytest.mark.parametrize("M,N,K", [(128, 256, 512), (128, 256, 1024), (256, 512, 1536), (128, 256, 2048),
                                   (136, 320, 2560), (264, 576, 3072), (128, 256, 3584), (512, 768, 4096),
                                   (1000, 1088, 4608), (128, 64, 5120), (512, 512, 8192)])
@pytest.mark.parametrize("dtype_c", ["f32", "bf16"])
def test_mxfp4_stream_direct_b(gpu, M, N, K, dtype_c):
    """MXFP4 with B pre-shuffled (payload in step order, e8m0 plane in lane order) and loaded
    straight into MFMA operands: 128 x 256 tiles, four waves.  K-step counts 2, 4, 6 (no steady
    group), 8 (one steady group exactly), 10, 12, 14, 16, 18, 20, 32; edge tiles in M (multiple
    of 8) and N (multiple of 64).  Scales differ from row to row and block to block, so a wrong
    scale byte (row, block, tile or half) shows.  Against the oracle, and the same bits as the
    kernel that takes B row-major through LDS."""
    from aster_amd.kittens_helpers import shuffle_scales_e8m0_lanes, shuffle_weight_bytes
    rng = np.random.default_rng(K + M)
    xa = rng.standard_normal((M, K)).astype(np.float32) * (2.0 ** rng.integers(-3, 4, (M, 1))).astype(np.float32)
    xb = rng.standard_normal((N, K)).astype(np.float32) * (2.0 ** rng.integers(-3, 4, (N, 1))).astype(np.float32)
    xa.reshape(M, K // 32, 32)[:] *= (2.0 ** rng.integers(-2, 3, (M, K // 32, 1))).astype(np.float32)
    xb.reshape(N, K // 32, 32)[:] *= (2.0 ** rng.integers(-2, 3, (N, K // 32, 1))).astype(np.float32)
    a, mxa = F.quantize_mxfp4(xa)
    b, mxb = F.quantize_mxfp4(xb)
    bias = rng.standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, shuffle_weight_bytes(b), M, N, K, "mxfp4", dtype_c, bias=bias, mx_a=mxa,
                         mx_b=shuffle_scales_e8m0_lanes(mxb), operand_path="direct_b_k8")
    assert name == f"streamdb_mxfp4_128x256_w1x4_{dtype_c}"
    check(out, G.gemm_mxfp4(a, mxa, b, mxb, out_dtype=_DT[dtype_c], bias=bias), dtype_c, N,
          bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    lds_out, lds_name = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, bias=bias, mx_a=mxa, mx_b=mxb,
                                 family=_capi.KERNEL_TILE)
    if lds_name.startswith("stream_mxfp4"):   # the same products in the same order
        assert np.array_equal(out.view(np.uint8), lds_out.view(np.uint8))
    # A's e8m0 plane in lane order (groups of 128 rows, padded): one 16-byte load per wave and
    # K-step instead of the pass through LDS; the same bits
    from aster_amd.kittens_helpers import shuffle_scales_e8m0_lanes128
    sal, sal_name = run_gemm(a, shuffle_weight_bytes(b), M, N, K, "mxfp4", dtype_c, bias=bias,
                             mx_a=shuffle_scales_e8m0_lanes128(mxa), mx_b=shuffle_scales_e8m0_lanes(mxb),
                             operand_path="direct_b_k8", mx_a_layout="lanes128")
    assert sal_name == f"streamdb_mxfp4_128x256_w1x4_sal_{dtype_c}"
    assert np.array_equal(sal.view(np.uint8), out.view(np.uint8))


def test_mxfp4_lane_order_activation_scales_are_refused_where_no_kernel_reads_them(gpu):
    with pytest.raises(_capi.AsterGemmError):      # row-major weights: the LDS kernels read rows
        AG.GemmPlan.create(512, 512, 4096, "mxfp4", "bf16", mx_a_layout="lanes128")
    with pytest.raises(_capi.AsterGemmError):      # not an MXFP4 problem
        AG.GemmPlan.create(512, 512, 4096, "bf16", "bf16", mx_a_layout="lanes128")
    p = AG.GemmPlan.create(512, 512, 4096, "mxfp4", "bf16", operand_path="direct_b_k8", mx_a_layout="lanes128")
    assert p.info.name.decode() == "streamdb_mxfp4_128x256_w1x4_sal_bf16"


def test_mxfp4_quantise_into_lane_order_then_gemm_full_size(gpu):
    """Configuration 5 at the size the bench times with everything made on the device: activations
    quantised straight into (payload, lane-order plane), weights quantised and pre-shuffled, GEMM
    through the lane-order kernel.  The plane equals the host shuffle of the row-major plane, and
    the product equals the row-major path's bit for bit and the oracle's on sampled rows."""
    from aster_amd.kittens_helpers import mx_lanes128_bytes, shuffle_scales_e8m0_lanes128
    from aster_amd.quantize import preshuffle_device, preshuffle_scales_a_device, quantize_mxfp4_device
    M, N, K = 4096, 14336, 4096
    rng = np.random.default_rng(5)
    xa = rng.standard_normal((M, K)).astype(np.float32)
    xb = rng.standard_normal((N, K)).astype(np.float32)
    a, mxa = F.quantize_mxfp4(xa)
    b, mxb = F.quantize_mxfp4(xb)
    bufs = {k: GpuBuffer(n) for k, n in dict(xa=xa.nbytes, xb=xb.nbytes, a=M * K // 2, b=N * K // 2,
                                             bs=N * K // 2, sa=mx_lanes128_bytes(M, K), sa2=mx_lanes128_bytes(M, K),
                                             sar=M * K // 32, sb=N * K // 32, sbs=N * K // 32, c=M * N * 2).items()}
    bufs["xa"].copy_from_host(xa)
    bufs["xb"].copy_from_host(xb)
    quantize_mxfp4_device(bufs["xa"].ptr_value, M, K, bufs["a"].ptr_value, bufs["sa"].ptr_value,
                          scales_layout="lanes128")
    quantize_mxfp4_device(bufs["xa"].ptr_value, M, K, bufs["a"].ptr_value, bufs["sar"].ptr_value)
    preshuffle_scales_a_device(bufs["sar"].ptr_value, bufs["sa2"].ptr_value, M, K)
    quantize_mxfp4_device(bufs["xb"].ptr_value, N, K, bufs["b"].ptr_value, bufs["sb"].ptr_value)
    preshuffle_device(bufs["b"].ptr_value, bufs["bs"].ptr_value, N, K, "mxfp4", "direct_b_k8",
                      d_mx_src=bufs["sb"].ptr_value, d_mx_dst=bufs["sbs"].ptr_value)
    got_sa, got_sa2 = np.empty(mx_lanes128_bytes(M, K), np.uint8), np.empty(mx_lanes128_bytes(M, K), np.uint8)
    bufs["sa"].copy_to_host(got_sa)
    bufs["sa2"].copy_to_host(got_sa2)
    assert np.array_equal(got_sa, shuffle_scales_e8m0_lanes128(mxa))
    assert np.array_equal(got_sa2, got_sa)
    out = np.zeros((M, N), np.uint16)
    plan = AG.GemmPlan.create(M, N, K, "mxfp4", "bf16", operand_path="direct_b_k8", mx_a_layout="lanes128")
    assert plan.info.name.decode() == "streamdb_mxfp4_128x256_w1x4_sal_bf16"
    print("launch", plan.info.name.decode(), flush=True)
    plan.run(bufs["a"].ptr_value, bufs["bs"].ptr_value, bufs["c"].ptr_value, mx_a=bufs["sa"].ptr_value,
             mx_b=bufs["sbs"].ptr_value)
    bufs["c"].copy_to_host(out)
    for bf in bufs.values():
        bf.free()
    rows, cols = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm_mxfp4(a[rows], mxa[rows], b, mxb, out_dtype=G.BF16), "bf16", N)
    check(out[:, cols], G.gemm_mxfp4(a, mxa, b[cols], mxb[cols], out_dtype=G.BF16), "bf16", len(cols))
    plain, _ = run_gemm(a, b, M, N, K, "mxfp4", "bf16", mx_a=mxa, mx_b=mxb)
    assert np.array_equal(out, plain)


def test_mxfp4_stream_direct_b_full_size_row_sample(gpu):
    # configuration 5 at the size the bench times, weights pre-shuffled
    from aster_amd.kittens_helpers import shuffle_scales_e8m0_lanes, shuffle_weight_bytes
    M, N, K = 4096, 14336, 4096
    a, b, ex = operands(M, N, K, "mxfp4", a_std=1.0, b_std=1.0)
    out, name = run_gemm(a, shuffle_weight_bytes(b), M, N, K, "mxfp4", "bf16", mx_a=ex["mx_a"],
                         mx_b=shuffle_scales_e8m0_lanes(ex["mx_b"]), operand_path="direct_b_k8")
    assert name == "streamdb_mxfp4_128x256_w1x4_bf16"
    rows, cols = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm_mxfp4(a[rows], ex["mx_a"][rows], b, ex["mx_b"], out_dtype=G.BF16), "bf16", N)
    check(out[:, cols], G.gemm_mxfp4(a, ex["mx_a"], b[cols], ex["mx_b"][cols], out_dtype=G.BF16),
          "bf16", len(cols))
    plain, _ = run_gemm(a, b, M, N, K, "mxfp4", "bf16", **ex)
    assert np.array_equal(out, plain)


@pytest.mark.parametrize("M,N,K", [(128, 256, 128), (128, 256, 256), (136, 272, 384), (128, 256, 512),
                                   (256, 512, 640), (128, 256, 896), (128, 256, 1024), (264, 528, 1152),
                                   (128, 256, 1408), (512, 768, 1536), (128, 256, 1664), (1000, 1072, 2048),
                                   (128, 64, 4096), (512, 512, 8192)])
@pytest.mark.parametrize("dtype_c", ["f32", "bf16"])
def test_fp8_stream_direct_b(gpu, M, N, K, dtype_c):
    """fp8 with B pre-shuffled into step order and loaded straight into MFMA operands: 128 x 256
    tiles, four waves, every load of the K loop counted by hand.  K-step counts 1..7 (no steady
    group: every wait is for all loads), 8 (the first group and the last), 9, 11, 13 (first
    group, then trips that wait for all), 12, 16, 32, 64 (steady groups between the first and
    the last); edge tiles in M (multiple of 8) and N (multiple of 16).  Against the oracle, and
    the same bits as the kernel that takes B row-major through LDS."""
    from aster_amd.kittens_helpers import shuffle_weight_bytes
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=K + M, b_std=0.05)
    bias = np.random.default_rng(K).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, shuffle_weight_bytes(b), M, N, K, "fp8_e4m3", dtype_c, bias=bias,
                         operand_path="direct_b_k8", **ex)
    assert name == f"streamdb_fp8_128x256_w1x4_{dtype_c}"
    check(out, G.gemm_fp8(a, b, ex["scale_a"], ex["scale_b"], out_dtype=_DT[dtype_c], bias=bias), dtype_c, N,
          bar=1e-4 if dtype_c == "f32" else REL_L2_BAR)
    lds_out, lds_name = run_gemm(a, b, M, N, K, "fp8_e4m3", dtype_c, bias=bias, family=_capi.KERNEL_TILE,
                                 wg_tile=(256, 256), **ex)
    assert lds_name.startswith("stream_fp8_256x256")   # the same products in the same order
    assert np.array_equal(out.view(np.uint8), lds_out.view(np.uint8))


def test_fp8_stream_direct_b_full_size_row_sample(gpu):
    # configuration 3 at the size the bench times, weights pre-shuffled: sampled rows against the
    # oracle, every element against the kernel that takes B row-major
    from aster_amd.kittens_helpers import shuffle_weight_bytes
    M = N = K = 8192
    a, b, ex = operands(M, N, K, "fp8_e4m3", a_std=1.0, b_std=1.0)
    out, name = run_gemm(a, shuffle_weight_bytes(b), M, N, K, "fp8_e4m3", "bf16", operand_path="direct_b_k8",
                         **ex)
    assert name == "streamdb_fp8_128x256_w1x4_bf16"
    rows, _ = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm_fp8(a[rows], b, ex["scale_a"], ex["scale_b"], out_dtype=G.BF16), "bf16", N)
    plain, _ = run_gemm(a, b, M, N, K, "fp8_e4m3", "bf16", **ex)
    assert np.array_equal(out, plain)


def test_stream_direct_b_k8_full_size_row_sample(gpu, big):
    from aster_amd.kittens_helpers import shuffle_weight_k8
    M, N, K, a, b = big
    out, name = run_gemm(a, shuffle_weight_k8(b), M, N, K, "bf16", "bf16", operand_path="direct_b_k8")
    assert name == "streamdb_bf16_128x256_w1x4_bf16"
    rows, cols = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm(a[rows], b, G.BF16, G.BF16), "bf16", N)
    check(out[:, cols], G.gemm(a, b[cols], G.BF16, G.BF16), "bf16", len(cols))
    out2, _ = run_gemm(a, shuffle_weight_k8(b), M, N, K, "bf16", "bf16", operand_path="direct_b_k8")
    assert np.array_equal(out, out2)


def test_the_reference_best_mapping_is_honoured_as_it_stands(gpu, tmp_path):
    # the mapping of the reference's best gfx950 label (128 x 256 workgroup tile = 8 x 16 MFMA
    # tiles, four waves in a 1 x 4 grid, B pre-shuffled and loaded straight into operands) selects
    # a kernel of exactly that geometry; nothing of the request is reported as dropped
    M, N, K = 1024, 1536, 1024
    cfg = make_instance(M, N, K, wg_tile=(128, 256), waves=(1, 4), operand_path=OperandPath.DIRECT_B)
    path, _ = AG.compile_gemm(cfg, str(tmp_path / "k.hsaco"))
    desc = json.load(open(path))
    assert desc["kernel"] == "streamdb_bf16_128x256_w1x4_bf16", desc
    assert desc["mapping_honoured"] is True and not desc.get("mapping_not_honoured")
    assert desc["grid"] == (M // 128) * (N // 256) and desc["block"] == 256
    a, b, _ = operands(M, N, K, "bf16")
    c_flat, times = AG.execute_gemm_hsaco(cfg, path, 2, a, b)
    check(c_flat.reshape(M, N), G.gemm(a, b, G.BF16, G.BF16), "bf16", N)


def test_direct_b_mapping_through_the_harness_seam(gpu, tmp_path):
    # a DIRECT_B mapping on a compute-bound shape: compile_gemm selects the kernel that reads
    # pre-shuffled B, execute_gemm_hsaco shuffles the row-major B it is given in that kernel's order
    cfg = make_instance(512, 768, 640, operand_path=OperandPath.DIRECT_B)
    path, asm = AG.compile_gemm(cfg, str(tmp_path / "k.hsaco"))
    desc = json.load(open(path))
    assert desc["kernel"].startswith("streamdb_") and desc["operand_path"] == "direct_b_k8"
    assert desc["mapping_honoured"] is True
    a, b, _ = operands(512, 768, 640, "bf16")
    c_flat, times = AG.execute_gemm_hsaco(cfg, path, 3, a, b)
    assert len(times) == 3
    check(c_flat.reshape(512, 768), G.gemm(a, b, G.BF16, G.BF16), "bf16", 768)


@pytest.mark.parametrize("dtype_ab,K", [("fp8_e4m3", 4096), ("mxfp4", 8192)])
def test_direct_b_mapping_of_a_decode_shape_with_byte_operands(gpu, tmp_path, dtype_ab, K):
    # the same seam for fp8 / MXFP4 on a decode shape: the DIRECT_B mapping selects the kernel that
    # reads the payload in step order, execute_gemm_hsaco shuffles the row-major payload (and the
    # MXFP4 scale plane) it is given
    M, N = 16, 528
    cfg = make_instance(M, N, K, dtype_ab=dtype_ab, dtype_c="f32", wg_tile=(16, 16), waves=(1, 1),
                        operand_path=OperandPath.DIRECT_B)
    path, asm = AG.compile_gemm(cfg, str(tmp_path / "k.hsaco"))
    desc = json.load(open(path))
    assert desc["kernel"].startswith("skinnyd_") and desc["operand_path"] == "direct_b"
    a, b, ex = operands(M, N, K, dtype_ab, seed=91, b_std=0.05)
    c_flat, times = AG.execute_gemm_hsaco(cfg, path, 2, a, b, **ex)
    want = G.gemm(a, b, _DT[dtype_ab], G.F32, **ex)
    check(c_flat.reshape(M, N), want, "f32", N, bar=1e-4)


def test_direct_b_mapping_of_a_compute_bound_fp8_shape(gpu, tmp_path):
    # the reference's best mapping (128 x 256, waves 1 x 4, DIRECT_B) with fp8 operands: the stream
    # kernel that loads the pre-shuffled payload straight into MFMA operands
    M, N, K = 512, 768, 1152
    cfg = make_instance(M, N, K, dtype_ab="fp8_e4m3", dtype_c="f32", wg_tile=(128, 256), waves=(1, 4),
                        operand_path=OperandPath.DIRECT_B)
    path, asm = AG.compile_gemm(cfg, str(tmp_path / "k.hsaco"))
    desc = json.load(open(path))
    assert desc["kernel"] == "streamdb_fp8_128x256_w1x4_f32" and desc["operand_path"] == "direct_b_k8"
    assert desc["mapping_honoured"] is True
    a, b, ex = operands(M, N, K, "fp8_e4m3", seed=93, b_std=0.05)
    c_flat, times = AG.execute_gemm_hsaco(cfg, path, 2, a, b, **ex)
    check(c_flat.reshape(M, N), G.gemm(a, b, G.FP8_E4M3, G.F32, **ex), "f32", N, bar=1e-4)


# ---- direct_ab: A and B both pre-shuffled, neither through LDS ---------------------------------

@pytest.mark.parametrize("M,N,K", [(16, 16, 32), (128, 256, 64), (128, 256, 96), (144, 272, 128),
                                   (256, 512, 160), (512, 768, 224), (1008, 1040, 256),
                                   (128, 1024, 576), (2048, 2048, 4096)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "bf16"), ("f16", "f32"), ("bf16", "f16")])
@pytest.mark.parametrize("tile,waves", [((128, 256), "1x4"), ((256, 256), "2x2")])
def test_direct_ab(gpu, M, N, K, dtype_ab, dtype_c, tile, waves):
    """Both operands in the reference's `shuffle_weight` order, straight into MFMA operands
    (reference template: gemm_16x32_f16_k_loop_helpers_direct_ab.mlir; execute side
    test_perf_001_gemm_fp16_weak_scaled.py:252-254).  Chunk-column counts 1, 2, 3, 4 (one whole
    ring of the 128 x 256 form), 5, 7, 8, 18, 128; edge tiles in M and N (multiples of 16); N(0,1)
    data, so a wrong lane or K order fails.  Both geometries: 128 x 64 per wave with a ring of four
    chunk columns, 128 x 128 per wave with a ring of three."""
    from aster_amd.kittens_helpers import shuffle_weight
    a, b, _ = operands(M, N, K, dtype_ab)
    bias = np.random.default_rng(4).standard_normal(N).astype(np.float32)
    out, name = run_gemm(shuffle_weight(a), shuffle_weight(b), M, N, K, dtype_ab, dtype_c, bias=bias,
                         operand_path="direct_ab", wg_tile=tile)
    assert name.startswith(f"directab_{dtype_ab}_{tile[0]}x{tile[1]}_w{waves}_")
    check(out, G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias), dtype_c, N)


def test_direct_ab_output_pitch_and_no_bias(gpu):
    from aster_amd.kittens_helpers import shuffle_weight
    M, N, K, ldc = 272, 528, 352, 540
    a, b, _ = operands(M, N, K, "bf16")
    out, _ = run_gemm(shuffle_weight(a), shuffle_weight(b), M, N, K, "bf16", "bf16", ldc=ldc,
                      operand_path="direct_ab")
    check(out, G.gemm(a, b, G.BF16, G.BF16), "bf16", N)
    assert (out[:, N:] == 0x7FC1).all()          # the padding of the rows is not written


def test_direct_ab_full_size_row_sample_with_device_preshuffle(gpu, big):
    """8192^3 with both operands shuffled on the device (`astergemm_preshuffle`, one call per
    operand); the device order equals the host's, rows and columns sampled against the oracle."""
    import torch
    from aster_amd import quantize as Q
    from aster_amd.kittens_helpers import shuffle_weight
    M, N, K, a, b = big
    dev = torch.device("cuda:0")
    ta = torch.from_numpy(a.view(np.int16)).to(dev)
    tb = torch.from_numpy(b.view(np.int16)).to(dev)
    sa, sb = torch.empty_like(ta), torch.empty_like(tb)
    tc = torch.zeros(M, N, dtype=torch.int16, device=dev)
    torch.cuda.synchronize()
    Q.preshuffle_device(ta.data_ptr(), sa.data_ptr(), M, K, "bf16", "direct_ab")
    Q.preshuffle_device(tb.data_ptr(), sb.data_ptr(), N, K, "bf16", "direct_ab")
    plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16", operand_path="direct_ab")
    assert plan.info.name.decode() == "directab_bf16_256x256_w2x2_bf16"
    print(f"launch {plan.info.name.decode()} M={M} N={N} K={K}", flush=True)
    plan.run(sa.data_ptr(), sb.data_ptr(), tc.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(sa[:64].cpu().numpy().view(np.uint16), shuffle_weight(a[:64]))
    out = tc.cpu().numpy().view(np.uint16)
    rows, cols = _sampled_rows_and_cols(M, N)
    check(out[rows], G.gemm(a[rows], b, G.BF16, G.BF16), "bf16", N)
    check(out[:, cols], G.gemm(a, b[cols], G.BF16, G.BF16), "bf16", len(cols))


def test_direct_ab_mapping_through_the_harness_seam(gpu, tmp_path):
    # a DIRECT_AB mapping: compile_gemm selects the kernel without LDS, execute_gemm_hsaco shuffles
    # the row-major A and B it is given (the reference's single point of truth)
    M, N, K = 512, 768, 640
    cfg = make_instance(M, N, K, wg_tile=(128, 256), waves=(1, 4), operand_path=OperandPath.DIRECT_AB)
    path, asm = AG.compile_gemm(cfg, str(tmp_path / "k.hsaco"))
    desc = json.load(open(path))
    assert desc["kernel"] == "directab_bf16_128x256_w1x4_bf16" and desc["operand_path"] == "direct_ab"
    assert desc["mapping_honoured"] is True and desc["lds_bytes"] == 0
    a, b, _ = operands(M, N, K, "bf16")
    c_flat, times = AG.execute_gemm_hsaco(cfg, path, 3, a, b)
    assert len(times) == 3
    check(c_flat.reshape(M, N), G.gemm(a, b, G.BF16, G.BF16), "bf16", N)
    # rows that do not fill 32-element chunks: the LDS kernels run and the descriptor says so
    cfg = make_instance(512, 768, 264, operand_path=OperandPath.DIRECT_AB)
    path, _ = AG.compile_gemm(cfg, str(tmp_path / "k2.hsaco"))
    desc = json.load(open(path))
    assert desc["operand_path"] == "lds"
    assert desc["mapping_not_honoured"]["operand_path"] == {"requested": "direct_ab", "kernel": "lds"}
    a, b, _ = operands(512, 768, 264, "bf16")
    c_flat, _ = AG.execute_gemm_hsaco(cfg, path, 1, a, b)
    check(c_flat.reshape(512, 768), G.gemm(a, b, G.BF16, G.BF16), "bf16", 768)


def test_direct_ab_is_refused_where_it_is_not_implemented(gpu):
    for kw in (dict(M=120, N=256, K=512), dict(M=128, N=264, K=512), dict(M=128, N=256, K=528)):
        with pytest.raises(_capi.AsterGemmError):
            AG.GemmPlan.create(kw["M"], kw["N"], kw["K"], "bf16", "bf16", operand_path="direct_ab")
    with pytest.raises(_capi.AsterGemmError):
        AG.GemmPlan.create(128, 256, 512, "fp8_e4m3", "bf16", operand_path="direct_ab")
    with pytest.raises(_capi.AsterGemmError):
        AG.GemmPlan.create(128, 256, 512, "bf16", "bf16", operand_path="direct_ab", lda=520)


def test_direct_b_is_refused_where_it_is_not_implemented(gpu):
    for kw in (dict(M=128, N=256, K=4096), dict(M=16, N=256, K=1024), dict(M=16, N=24, K=4096)):
        with pytest.raises(_capi.AsterGemmError):
            AG.GemmPlan.create(kw["M"], kw["N"], kw["K"], "bf16", "bf16", operand_path="direct_b")


# ---- linalg.matmul-shaped caller (B given K x N) ------------------------------------------

@pytest.mark.parametrize("M,N,K", [(32, 32, 32), (48, 200, 72), (512, 768, 256), (16, 1024, 2048)])
def test_linalg_matmul_kxn(gpu, M, N, K):
    # contrib/mlir-air/test/integration/test_linalg_matmul_e2e.py:52-75: seed 42, randn * 0.1,
    # B given K x N, rtol = atol = 1e-2
    from aster_amd.linalg import matmul
    np.random.seed(42)
    a = (np.random.randn(M, K) * 0.1).astype(np.float16)
    b_kxn = (np.random.randn(K, N) * 0.1).astype(np.float16)
    c = matmul(a, b_kxn)
    expected = a.astype(np.float32) @ b_kxn.astype(np.float32)
    np.testing.assert_allclose(c, expected, rtol=1e-2, atol=1e-2)
    assert G.rel_l2(c, expected) <= 1e-5
    with pytest.raises(ValueError):
        matmul(a, b_kxn[:-1])
    with pytest.raises(ValueError):
        matmul(a.astype(np.float32), b_kxn)


@pytest.mark.parametrize("M,N,K", [(264, 520, 512), (504, 1000, 1024), (1000, 264, 1536), (8, 8, 512)])
@pytest.mark.parametrize("dtype_c", ["bf16", "f32"])
@pytest.mark.parametrize("tile", [256, 128])
def test_mxfp4_stream_kernel_edge_tiles(gpu, M, N, K, dtype_c, tile):
    a, b, extra = operands(M, N, K, "mxfp4", seed=71, b_std=0.05)
    rng = np.random.default_rng(72)
    extra["mx_a"] = (extra["mx_a"].astype(np.int32) + rng.integers(-3, 4, extra["mx_a"].shape)).astype(np.uint8)
    extra["mx_b"] = (extra["mx_b"].astype(np.int32) + rng.integers(-3, 4, extra["mx_b"].shape)).astype(np.uint8)
    bias = rng.standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, "mxfp4", dtype_c, bias=bias, ldc=N + 16,
                         family=_capi.KERNEL_TILE, wg_tile=(tile, tile), **extra)
    assert name.startswith(f"stream_mxfp4_{tile}")
    want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[dtype_c], bias=bias)
    if M * N >= 4096:
        check(out, want, dtype_c, N, bar=1e-5 if dtype_c == "f32" else REL_L2_BAR)
    else:
        got, ref = G.output_to_f32(out[:, :N], _DT[dtype_c]), G.output_to_f32(want, _DT[dtype_c])
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-4 * np.abs(ref).max())
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (264, 520, 136), (504, 1000, 1016), (1000, 264, 7008),
                                   (2056, 1800, 256), (136, 128, 72)])
@pytest.mark.parametrize("dtype_ab,dtype_c", [("bf16", "bf16"), ("f16", "f32"), ("fp8_e4m3", "bf16"),
                                              ("fp8_e4m3", "f32")])
def test_stream_kernel_128_tiles_edges_and_k_tails(gpu, M, N, K, dtype_ab, dtype_c):
    if dtype_ab == "fp8_e4m3":
        K = (K + 15) // 16 * 16 * 2       # whole granules, and a few more K steps
    a, b, extra = operands(M, N, K, dtype_ab, seed=81, b_std=0.05)
    bias = np.random.default_rng(82).standard_normal(N).astype(np.float32)
    out, name = run_gemm(a, b, M, N, K, dtype_ab, dtype_c, bias=bias, ldc=N + 16,
                         family=_capi.KERNEL_TILE, wg_tile=(128, 128), **extra)
    assert name.startswith("stream_") and "128x128" in name
    if dtype_ab == "fp8_e4m3":
        want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[dtype_c], bias=bias)
        check(out, want, dtype_c, N, bar=REL_L2_BAR if dtype_c != "f32" else 1e-4)
    else:
        want = G.gemm(a, b, _DT[dtype_ab], _DT[dtype_c], bias=bias)
        check(out, want, dtype_c, N, bar=REL_L2_BAR if dtype_c != "f32" else 1e-5)
    pad = out[:, N:]
    assert np.isnan(pad).all() if dtype_c == "f32" else (pad == 0x7FC1).all()


# ---- seeded random shapes through AUTO selection ------------------------------------------------

def _random_cases(n_cases=96, seed=2024):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n_cases):
        dt = ("bf16", "f16", "fp8_e4m3", "mxfp4")[i % 4]
        kind = rng.integers(0, 4)
        if kind == 0:      # decode shapes
            M = int(rng.choice([1, 7, 16, 16, 17, 32, 33, 64]))
            N = int(rng.integers(1, 400)) * 8
            K = int(rng.choice([2048, 4096, 8192]))
        elif kind == 1:    # big enough for the 256 x 256 kernels, edges and K tails
            M = int(rng.integers(490, 540)) * 8
            N = int(rng.integers(490, 540)) * 8
            K = int(rng.integers(8, 40)) * 16
        elif kind == 2:    # mid-sized, any M and N
            M = int(rng.integers(65, 900))
            N = int(rng.integers(1, 900))
            K = int(rng.integers(4, 64)) * 16
        else:              # tiny
            M = int(rng.integers(1, 64))
            N = int(rng.integers(1, 64))
            K = int(rng.integers(1, 16)) * 16
        if dt == "mxfp4":
            K = max(256, (K + 255) // 256 * 256)
        if dt in ("bf16", "f16"):
            K = max(8, K // 8 * 8)
        out = ("f32", "bf16", "f16")[int(rng.integers(0, 3))]
        cases.append((dt, out, M, N, K, bool(rng.integers(0, 2)), int(rng.integers(0, 3)) * 8))
    return cases


@pytest.mark.parametrize("dt,out_dt,M,N,K,with_bias,pad", _random_cases())
def test_random_shapes_through_auto_selection(gpu, dt, out_dt, M, N, K, with_bias, pad):
    """Whatever kernel AUTO picks for a shape (stream with edge tiles and K tails, the four tile
    sizes, the skinny kernels), the result equals the oracle's; pad columns stay untouched."""
    a, b, extra = operands(M, N, K, dt, seed=1000 + M + N + K, b_std=0.05)
    bias = np.random.default_rng(5).standard_normal(N).astype(np.float32) if with_bias else None
    ldc = N + pad if pad else 0
    out, name = run_gemm(a, b, M, N, K, dt, out_dt, bias=bias, ldc=ldc, **extra)
    if dt == "fp8_e4m3":
        want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[out_dt], bias=bias)
    elif dt == "mxfp4":
        want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[out_dt], bias=bias)
    else:
        want = G.gemm(a, b, _DT[dt], _DT[out_dt], bias=bias)
    got, ref = G.output_to_f32(out[:, :N], _DT[out_dt]), G.output_to_f32(want, _DT[out_dt])
    assert not np.isnan(got).any(), name
    ulp = {"f32": 2.0 ** -20, "bf16": 2.0 ** -7, "f16": 2.0 ** -10}[out_dt]
    tol = 2 * ulp * np.abs(ref) + 2e-4 * np.abs(ref).max()
    assert np.all(np.abs(got - ref) <= tol), (name, float(np.abs(got - ref).max()))
    if M * N >= 4096:
        bar = REL_L2_BAR if out_dt != "f32" else (1e-4 if dt == "fp8_e4m3" else 1e-5)
        assert G.rel_l2(got, ref) <= bar, name
    if pad:
        tail = out[:, N:]
        assert np.isnan(tail).all() if out_dt == "f32" else (tail == 0x7FC1).all()


def _random_pre_shuffled_cases(n_cases=36, seed=77):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n_cases):
        dt = ("bf16", "f16", "fp8_e4m3", "mxfp4")[i % 4]
        M = int(rng.integers(1, 160)) * 8
        N = int(rng.integers(1, 24)) * 64
        K = int(rng.integers(1, 12)) * 512 if dt == "mxfp4" else int(rng.integers(1, 40)) * 128
        out = ("f32", "bf16", "f16")[int(rng.integers(0, 3))]
        cases.append((dt, out, M, N, K, bool(rng.integers(0, 2)), int(rng.integers(0, 3)) * 8))
    return cases


@pytest.mark.parametrize("dt,out_dt,M,N,K,with_bias,pad", _random_pre_shuffled_cases())
def test_random_shapes_with_pre_shuffled_weights(gpu, dt, out_dt, M, N, K, with_bias, pad):
    """The stream kernels that load pre-shuffled B straight into MFMA operands (operand_path
    direct_b_k8: 16-bit, fp8, MXFP4) on seeded random shapes with edge tiles in M and N and every
    residue of the K-step count: the oracle's result, pad columns untouched."""
    from aster_amd.kittens_helpers import shuffle_scales_e8m0_lanes, shuffle_weight_bytes, shuffle_weight_k8
    a, b, extra = operands(M, N, K, dt, seed=3000 + M + N + K, b_std=0.05)
    bias = np.random.default_rng(6).standard_normal(N).astype(np.float32) if with_bias else None
    dev = dict(extra)
    if dt in ("bf16", "f16"):
        b_dev = shuffle_weight_k8(np.ascontiguousarray(b).view(np.uint16))
    else:
        b_dev = shuffle_weight_bytes(b)
        if dt == "mxfp4":
            dev["mx_b"] = shuffle_scales_e8m0_lanes(extra["mx_b"])
    out, name = run_gemm(a, b_dev, M, N, K, dt, out_dt, bias=bias, ldc=N + pad if pad else 0,
                         operand_path="direct_b_k8", **dev)
    assert name.startswith("streamdb_")
    if dt == "fp8_e4m3":
        want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=_DT[out_dt], bias=bias)
    elif dt == "mxfp4":
        want = G.gemm_mxfp4(a, extra["mx_a"], b, extra["mx_b"], out_dtype=_DT[out_dt], bias=bias)
    else:
        want = G.gemm(a, b, _DT[dt], _DT[out_dt], bias=bias)
    got, ref = G.output_to_f32(out[:, :N], _DT[out_dt]), G.output_to_f32(want, _DT[out_dt])
    assert not np.isnan(got).any(), name
    ulp = {"f32": 2.0 ** -20, "bf16": 2.0 ** -7, "f16": 2.0 ** -10}[out_dt]
    tol = 2 * ulp * np.abs(ref) + 2e-4 * np.abs(ref).max()
    assert np.all(np.abs(got - ref) <= tol), (name, float(np.abs(got - ref).max()))
    bar = REL_L2_BAR if out_dt != "f32" else (1e-4 if dt == "fp8_e4m3" else 1e-5)
    assert G.rel_l2(got, ref) <= bar, name
    if pad:
        tail = out[:, N:]
        assert np.isnan(tail).all() if out_dt == "f32" else (tail == 0x7FC1).all()


def _random_direct_ab_cases(n_cases=24, seed=313):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n_cases):
        dt = ("bf16", "f16")[i % 2]
        big = i % 6 == 5          # enough tiles for the 256 x 256 form to be chosen
        M = int(rng.integers(225, 240) if big else rng.integers(1, 70)) * 16
        N = int(rng.integers(225, 240) if big else rng.integers(1, 70)) * 16
        K = int(rng.integers(1, 12 if big else 40)) * 32
        out = ("f32", "bf16", "f16")[int(rng.integers(0, 3))]
        cases.append((dt, out, M, N, K, bool(rng.integers(0, 2)), int(rng.integers(0, 3)) * 4))
    return cases


@pytest.mark.parametrize("dt,out_dt,M,N,K,with_bias,pad", _random_direct_ab_cases())
def test_random_shapes_with_both_operands_pre_shuffled(gpu, dt, out_dt, M, N, K, with_bias, pad):
    """operand_path direct_ab on seeded random shapes: edge tiles in M and N (multiples of 16),
    every residue of the chunk-column count against both ring depths, whichever of the two
    geometries AUTO takes; the oracle's result, pad columns untouched."""
    from aster_amd.kittens_helpers import shuffle_weight
    a, b, _ = operands(M, N, K, dt, seed=4000 + M + N + K, b_std=0.05)
    bias = np.random.default_rng(7).standard_normal(N).astype(np.float32) if with_bias else None
    out, name = run_gemm(shuffle_weight(np.ascontiguousarray(a).view(np.uint16)),
                         shuffle_weight(np.ascontiguousarray(b).view(np.uint16)), M, N, K, dt, out_dt,
                         bias=bias, ldc=N + pad if pad else 0, operand_path="direct_ab")
    assert name.startswith(f"directab_{dt}_")
    want = G.gemm(a, b, _DT[dt], _DT[out_dt], bias=bias)
    got, ref = G.output_to_f32(out[:, :N], _DT[out_dt]), G.output_to_f32(want, _DT[out_dt])
    assert not np.isnan(got).any(), name
    ulp = {"f32": 2.0 ** -20, "bf16": 2.0 ** -7, "f16": 2.0 ** -10}[out_dt]
    tol = 2 * ulp * np.abs(ref) + 2e-4 * np.abs(ref).max()
    assert np.all(np.abs(got - ref) <= tol), (name, float(np.abs(got - ref).max()))
    if M * N >= 4096:
        assert G.rel_l2(got, ref) <= (REL_L2_BAR if out_dt != "f32" else 1e-5), name
    if pad:
        tail = out[:, N:]
        assert np.isnan(tail).all() if out_dt == "f32" else (tail == 0x7FC1).all()


@pytest.mark.parametrize("M,N,K,dt", [(512, 768, 1024, "bf16"), (16, 520, 4096, "bf16"), (300, 200, 512, "fp8_e4m3")])
def test_tune_returns_a_runnable_variant_that_matches_the_oracle(gpu, M, N, K, dt):
    a, b, extra = operands(M, N, K, dt, seed=91, b_std=0.05)
    bufs = [GpuBuffer(x.nbytes) for x in (a, b)] + [GpuBuffer(M * N * 4)]
    bufs[0].copy_from_host(np.ascontiguousarray(a))
    bufs[1].copy_from_host(np.ascontiguousarray(b))
    kw = {}
    if dt == "fp8_e4m3":
        sc = GpuBuffer(8)
        sc.copy_from_host(np.array([extra["scale_a"], extra["scale_b"]], np.float32))
        kw = dict(scale_a=sc.ptr_value, scale_b=sc.ptr_value + 4)
    auto = AG.GemmPlan.create(M, N, K, dt, "f32")
    print(f"tune {dt} M={M} N={N} K={K}", flush=True)
    tuned = auto.tune(*(x.ptr_value for x in bufs), iters=5, **kw)
    assert tuned.config.variant == tuned.info.variant > 0 and tuned.tuned_ns > 0
    tuned.run(*(x.ptr_value for x in bufs), **kw)
    out = np.empty((M, N), np.float32)
    bufs[2].copy_to_host(out)
    if dt == "fp8_e4m3":
        want = G.gemm_fp8(a, b, extra["scale_a"], extra["scale_b"], out_dtype=G.F32)
    else:
        want = G.gemm(a, b, _DT[dt], G.F32)
    assert G.rel_l2(out, G.output_to_f32(want, G.F32)) <= 1e-4
    # restricting the family restricts the candidates
    only_tile = AG.GemmPlan.create(M, N, K, dt, "f32", family=_capi.KERNEL_TILE).tune(
        *(x.ptr_value for x in bufs), iters=3, **kw)
    assert only_tile.info.family == _capi.KERNEL_TILE


def test_library_loaded_before_pytorch_still_launches(gpu):
    """A process that loads the library first and imports PyTorch afterwards must end up with one
    HIP runtime: with two, the one initialised second reports that it finds no device at the
    first launch.  Fresh process: library, then torch, then a GEMM on torch-owned memory."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("from aster_amd import _capi, gemm as AG\n"
            "_capi.load()\n"
            "import torch\n"
            "a = torch.ones(256, 512, dtype=torch.bfloat16, device='cuda:0')\n"
            "b = torch.ones(384, 512, dtype=torch.bfloat16, device='cuda:0')\n"
            "c = torch.zeros(256, 384, dtype=torch.bfloat16, device='cuda:0')\n"
            "torch.cuda.synchronize()\n"
            "p = AG.GemmPlan.create(256, 384, 512, 'bf16', 'bf16')\n"
            "print('launch', p.info.name.decode(), flush=True)\n"
            "p.run(a.data_ptr(), b.data_ptr(), c.data_ptr())\n"
            "torch.cuda.synchronize()\n"
            "assert bool((c == 512).all()), c\n"
            "print('one runtime, launch ok')\n")
    out = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "launch ok" in out.stdout, out.stderr[-2000:]
