"""Layout algebra, swizzles, B pre-shuffle and the cooperative split."""
import ctypes
import itertools
import os
import math

import numpy as np
import pytest

from aster_amd import _capi
from aster_amd.coop import coop_2d_split, coop_wave_start
from aster_amd.kittens_helpers import shuffle_weight, unshuffle_weight
from aster_amd.layout import (TILE_LDS_SWIZZLE, Layout, Swizzle, delinearize, flatten_nested,
                              linearize, make_layout, product, suffix_product, tile)
from oracle import layouts as OL


def test_int_tuple_helpers():
    assert flatten_nested(((1, 2), 3, [4, (5,)])) == (1, 2, 3, 4, 5)
    assert flatten_nested(7) == (7,)
    assert product((2, 3, 4)) == 24 and product(5) == 5
    assert suffix_product((2, 3, 4)) == (12, 4, 1) and suffix_product(9) == 1
    assert delinearize(7, (4, 3)) == (2, 1)
    assert linearize((3, 1), (1, 4)) == 7
    for idx in range(24):
        assert linearize(delinearize(idx, (2, 3, 4)), suffix_product((2, 3, 4))) == idx


def test_layout_call_and_properties():
    l = Layout((4, 16), (16, 64))
    assert l(0) == 0 and l(1) == 64 and l(16) == 16 and l(17) == 80
    assert Layout((4, 16)).strides == (16, 1)
    assert Layout(8)(3) == 3
    assert l.size() == 64 and len(l) == 2 and l.is_flat and l.flat_sizes == (4, 16)
    assert not Layout(((2, 2), 4), ((1, 2), 4)).is_flat
    assert l == Layout((4, 16), (16, 64)) and l != Layout((4, 16))
    assert make_layout(Layout(4, 1), Layout(8, 4)) == Layout((4, 8), (1, 4))


def test_tile():
    t = tile(Layout((64, 32), (64, 2)), (16, 8))
    assert t.sizes == (4, 4, 16, 8) and t.strides == (1024, 16, 64, 2)
    h = tile(Layout((64,), (2,)), ((4, 2),))
    assert h.sizes == (2, 8, 4) and h.strides == (8, 16, 2)
    with pytest.raises(AssertionError):
        tile(Layout((10,), (1,)), (4,))


@pytest.mark.parametrize("sw", [Swizzle(3, 3, 4), Swizzle(2, 4, 4), TILE_LDS_SWIZZLE])
def test_swizzle_is_an_involution_and_keeps_low_bits(sw):
    span = 1 << (sw.base + sw.shift + sw.bits)
    image = [sw(o) for o in range(span)]
    assert sorted(image) == list(range(span))
    assert all(sw(sw(o)) == o for o in range(span))
    assert all((sw(o) ^ o) & ((1 << sw.base) - 1) == 0 for o in range(span))
    assert all(sw(o) == OL.swizzle(o, sw.bits, sw.base, sw.shift) for o in range(span))


def test_swizzle_3_3_4_is_the_mlir_16x64_formula():
    sw = Swizzle(3, 3, 4)
    for row in range(16):
        for byte in range(64):
            assert sw(row * 64 + byte) == OL.lds_swizzled_addr_16x64_b(0, row, byte)


def test_tile_lds_swizzle_matches_kernel_formula_and_is_conflict_free():
    for row in range(32):
        for g in range(8):
            assert TILE_LDS_SWIZZLE(row * 128 + g * 16) == OL.tile_lds_offset(row, g)
    # A ds_read_b128 serves 16 lanes at a time: 16 rows x one K granule must land
    # in 16 distinct 16-byte bank groups (64 banks x 4 B).
    for row0 in (0, 16):
        for g in range(8):
            offs = [OL.tile_lds_offset(row0 + i, g) for i in range(16)]
            assert len(set(OL.bank_groups_16B(offs))) == 16
    # without the swizzle the same access is an 8-way conflict
    assert len(set(OL.bank_groups_16B([i * 128 for i in range(16)]))) == 2


def test_mfma_fragment_maps_cover_the_tile():
    a = {(OL.mfma_index_a_16x16_f16(l)[0], OL.mfma_index_a_16x16_f16(l)[1] + e)
         for l in range(64) for e in range(4)}
    assert a == set(itertools.product(range(16), range(16)))
    f8 = {(OL.mfma_index_a_16x16_fp8(l)[0], OL.mfma_index_a_16x16_fp8(l)[1] + e)
          for l in range(64) for e in range(8)}
    assert f8 == set(itertools.product(range(16), range(32)))
    c = {(OL.mfma_index_c_16x16_f32(l)[1] + r, OL.mfma_index_c_16x16_f32(l)[0])
         for l in range(64) for r in range(4)}
    assert c == set(itertools.product(range(16), range(16)))
    # element (r, c) of the C tile is owned by lane 16 * (r // 4) + c
    for l in range(64):
        col, rb = OL.mfma_index_c_16x16_f32(l)
        assert l == 16 * (rb // 4) + col


@pytest.mark.parametrize("N,K", [(16, 32), (32, 64), (48, 96)])
def test_shuffle_weight(N, K):
    B = np.arange(N * K, dtype=np.uint16).reshape(N, K)
    S = shuffle_weight(B)
    assert np.array_equal(S, OL.shuffle_weight(B))
    assert np.array_equal(np.sort(S.reshape(-1)), B.reshape(-1))
    assert np.array_equal(unshuffle_weight(S), B)
    # the docstring's lane property: lane d of block (nb, kb) reads 8 contiguous
    # elements = B[nb*16 + d%16, kb*32 + kh*16 + (d//16)*4 + 0..3], kh = 0, 1
    flat = S.reshape(-1)
    for nb in range(N // 16):
        for kb in range(K // 32):
            for d in range(64):
                base = (nb * (K // 32) + kb) * 512 + d * 8
                for kh in range(2):
                    want = B[nb * 16 + d % 16, kb * 32 + kh * 16 + (d // 16) * 4:][:4]
                    assert np.array_equal(flat[base + kh * 4: base + kh * 4 + 4], want)
    # the C-ABI host routine gives the same bytes
    out = np.empty_like(B)
    _capi.check(_capi.load().astergemm_shuffle_weight_16(B.ctypes.data, out.ctypes.data, N, K))
    assert np.array_equal(out, S)


def test_shuffle_weight_k8_is_the_16x16x32_operand_order():
    from aster_amd.kittens_helpers import shuffle_weight_k8, unshuffle_weight_k8
    N, K = 48, 128
    B = np.arange(N * K, dtype=np.uint16).reshape(N, K)
    S = shuffle_weight_k8(B)
    assert np.array_equal(np.sort(S.reshape(-1)), B.reshape(-1))
    assert np.array_equal(unshuffle_weight_k8(S), B)
    # lane d of block (nb, kb) reads 8 contiguous elements = B[nb*16 + d%16, kb*32 + (d//16)*8 + 0..7]:
    # the K positions lane d of a wave feeds to v_mfma_f32_16x16x32 (k = 8 * (lane / 16) .. + 7,
    # the 16-bit form of the reference's fp8 fragment map, indexing.mlir:202-218)
    flat = S.reshape(-1)
    for nb in range(N // 16):
        for kb in range(K // 32):
            for d in range(64):
                base = (nb * (K // 32) + kb) * 512 + d * 8
                want = B[nb * 16 + d % 16, kb * 32 + (d // 16) * 8:][:8]
                assert np.array_equal(flat[base: base + 8], want)
    out = np.empty_like(B)
    _capi.check(_capi.load().astergemm_shuffle_weight_k8_16(B.ctypes.data, out.ctypes.data, N, K))
    assert np.array_equal(out, S)
    # it differs from the reference's order exactly in the K pairing inside a 32-wide block
    assert not np.array_equal(S, shuffle_weight(B))
    assert _capi.load().astergemm_shuffle_weight_k8_16(B.ctypes.data, out.ctypes.data, 15, 32) == -22


def test_shuffle_weight_rejects_bad_shapes():
    with pytest.raises(AssertionError):
        shuffle_weight(np.zeros((15, 32), np.float16))
    with pytest.raises(AssertionError):
        shuffle_weight(np.zeros((16, 48), np.float16))
    z = np.zeros((15, 32), np.uint16)
    assert _capi.load().astergemm_shuffle_weight_16(z.ctypes.data, z.ctypes.data, 15, 32) == -22


def test_coop_2d_split_bruteforce():
    for num_tiles in range(1, 33):
        for num_waves in (1, 2, 4, 8):
            for kt in range(1, 5):
                ws, wk, cs, ck = coop_2d_split(num_tiles, num_waves, kt)
                assert ws * wk == num_waves
                assert cs == math.ceil(num_tiles / ws) and ck == math.ceil(kt / wk)
                waste = ws * wk * cs * ck - num_tiles * kt
                for d in (d for d in range(1, num_waves + 1) if num_waves % d == 0):
                    other = num_waves * math.ceil(num_tiles / d) * math.ceil(kt / (num_waves // d))
                    assert waste <= other - num_tiles * kt
                covered = set()
                for w in range(num_waves):
                    s0 = coop_wave_start(w // wk, cs, num_tiles)
                    k0 = coop_wave_start(w % wk, ck, kt)
                    covered |= {(s, k) for s in range(s0, s0 + cs) for k in range(k0, k0 + ck)}
                assert covered >= set(itertools.product(range(num_tiles), range(kt)))
    assert coop_2d_split(8, 4, 1) == (4, 1, 2, 1)
    assert coop_2d_split(2, 8, 2) == (4, 2, 1, 1)


def test_make_coop_load_plan_covers_the_workgroup_tile_with_clamped_starts():
    from aster_amd.coop import make_coop_load_plan
    from aster_amd.layout import Layout

    # the reference's shape of use: tiles of 1 KiB in LDS, 16 rows of a row-major operand in
    # global memory, kt K tiles of 64 bytes each
    for num_tiles in (1, 3, 8, 12, 16):
        for kt in (1, 2, 4):
            for num_waves in (1, 2, 4, 8):
                g = Layout((num_tiles, kt), (16 * 8192, 64))
                l = Layout((num_tiles, kt), (kt * 1024, 1024))
                ws, wk, cs, ck = coop_2d_split(num_tiles, num_waves, kt)
                seen = set()
                for w in range(num_waves):
                    plan = make_coop_load_plan(w, num_waves=num_waves, wg_tile_global=g, wg_tile_lds=l)
                    assert plan.global_layout.sizes == (cs, ck) == plan.lds_layout.sizes
                    assert plan.unroll_axes == ("s", "k")
                    # clamped start in tile units, then the layout's strides (coop.py:77-83)
                    s0 = coop_wave_start(w // wk, cs, num_tiles)
                    k0 = coop_wave_start(w % wk, ck, kt)
                    assert plan.global_wave_off == s0 * 16 * 8192 + k0 * 64
                    assert plan.lds_wave_off == s0 * kt * 1024 + k0 * 1024
                    for go, lo in plan.transfers():
                        # global and LDS offsets name the same tile
                        s, k = divmod(lo, kt * 1024)[0], (lo % (kt * 1024)) // 1024
                        assert go == s * 16 * 8192 + k * 64 and s < num_tiles and k < kt
                        seen.add((s, k))
                assert seen == set(itertools.product(range(num_tiles), range(kt)))
    # hand-evaluated: 8 tiles, 4 waves, 1 K tile -> two adjacent tiles per wave; wave 3 starts at 6
    plan = make_coop_load_plan(3, num_waves=4, wg_tile_global=Layout((8, 1), (100, 7)),
                               wg_tile_lds=Layout((8, 1), (1024, 1024)))
    assert plan.transfers() == [(600, 6144), (700, 7168)]
    # 3 tiles on 4 waves: the split is (1 x 4) over K?  kt = 1, so ws = 4 wastes one wave, which
    # redoes the last tile instead of running past the end
    plans = [make_coop_load_plan(w, num_waves=4, wg_tile_global=Layout((3, 1), (10, 1)),
                                 wg_tile_lds=Layout((3, 1), (1, 1))) for w in range(4)]
    assert [p.global_wave_off for p in plans] == [0, 10, 20, 20]
    with pytest.raises(AssertionError):
        make_coop_load_plan(0, num_waves=2, wg_tile_global=Layout((4, 1), (1, 1)),
                            wg_tile_lds=Layout((4, 2), (2, 1)))
    with pytest.raises(ValueError):
        make_coop_load_plan(4, num_waves=4, wg_tile_global=Layout((4, 1), (1, 1)),
                            wg_tile_lds=Layout((4, 1), (1, 1)))


@pytest.mark.parametrize("tile_rows,num_waves", [(256, 8), (256, 4), (128, 4)])
def test_stream_kernel_staging_is_the_interleaved_coop_plan(tile_rows, num_waves):
    """What the stream kernels do (gemm_stream_kernel.hpp: LH = BM / 8 / NW transfers per wave
    and ring slot, transfer j of wave w from operand rows (j * NW + w) * 8 to LDS offset
    (j * NW + w) * 8 * 128 of the slot) is the plan `coop_2d_split` gives for BM / 8 tiles of
    8 rows, one K tile, interleaved over the waves."""
    from aster_amd.coop import stream_kernel_load_plan

    ld = 16384
    lh = tile_rows // 8 // num_waves
    assert coop_2d_split(tile_rows // 8, num_waves, 1) == (num_waves, 1, lh, 1)
    everything = []
    for w in range(num_waves):
        plan = stream_kernel_load_plan(w, tile_rows=tile_rows, num_waves=num_waves, ld_bytes=ld)
        assert plan.global_layout.sizes == (lh, 1)
        kernel = [((j * num_waves + w) * 8 * ld, (j * num_waves + w) * 8 * 128) for j in range(lh)]
        assert plan.transfers() == kernel
        everything += kernel
    # the slot is filled exactly once: every 1 KiB of it, every 8-row group of the tile
    assert sorted(lo for _, lo in everything) == [t * 1024 for t in range(tile_rows // 8)]
    assert sorted(go for go, _ in everything) == [t * 8 * ld for t in range(tile_rows // 8)]


def test_stream_kernels_are_compiled_from_the_coop_plan():
    """The header the stream kernels take LH, their operand rows and their LDS offsets from is the
    text the plan generator writes (the build rewrites it before compiling), its constants are
    the plan's, and no kernel source restates the staging formula."""
    import glob
    import re
    from aster_amd.build import CSRC, PLAN_HEADER
    from aster_amd.coop import STREAM_PLAN_CONFIGS, stream_kernel_load_plan, stream_load_plan_header
    with open(PLAN_HEADER) as f:
        text = f.read()
    assert text == stream_load_plan_header()
    for rows, nw in STREAM_PLAN_CONFIGS:
        body = text[text.index(f"struct StreamLoadPlan<{rows}, {nw}>"):]
        body = body[:body.index("};")]
        const = {k: int(v) for k, v in re.findall(r"static constexpr int (\w+) = (\d+);", body)}
        for w in range(nw):
            plan = stream_kernel_load_plan(w, tile_rows=rows, num_waves=nw, ld_bytes=4096)
            assert const["LH"] == plan.global_layout.sizes[0]
            for j, (go, lo) in enumerate(plan.transfers()):
                tile = w * const["WAVE_STEP_TILES"] + j * const["XFER_STEP_TILES"]
                assert go == tile * const["TILE_ROWS"] * 4096 and lo == tile * const["TILE_LDS_BYTES"]
    for path in glob.glob(os.path.join(CSRC, "gemm_stream*_kernel.hpp")):
        with open(path) as f:
            src = f.read()
        assert "StreamLoadPlan<BM, NW>" in src, path
        assert "j * NW + wave" not in src and "BM / 8 / NW" not in src, path


def test_shuffle_weight_bytes_is_the_operand_order_of_the_16x16x128_mfma():
    # lane 16 q + n of the KiB (row block nb, step s, half u) holds bytes [(4u + q) * 16, + 16) of
    # row 16 nb + n, step s; the C-ABI function writes the same bytes; the inverse restores them
    import ctypes
    from aster_amd import _capi
    from aster_amd.kittens_helpers import (shuffle_scales_e8m0, shuffle_weight_bytes,
                                           unshuffle_scales_e8m0, unshuffle_weight_bytes)
    rng = np.random.default_rng(5)
    N, rb = 48, 384
    b = rng.integers(0, 256, (N, rb)).astype(np.uint8)
    sh = shuffle_weight_bytes(b)
    flat = sh.reshape(-1)
    steps = rb // 128
    for (nb, st, u, q, n) in ((0, 0, 0, 0, 0), (2, 1, 1, 3, 15), (1, 2, 0, 2, 7), (2, 2, 1, 0, 9)):
        at = ((nb * steps + st) * 2 + u) * 1024 + (16 * q + n) * 16
        assert np.array_equal(flat[at:at + 16], b[16 * nb + n, st * 128 + (4 * u + q) * 16:][:16])
    assert np.array_equal(unshuffle_weight_bytes(sh), b)
    out = np.empty_like(b)
    _capi.check(_capi.load().astergemm_shuffle_weight_8(b.ctypes.data, out.ctypes.data, N, rb))
    assert np.array_equal(out, sh)
    with pytest.raises(AssertionError):
        shuffle_weight_bytes(b[:40])
    with pytest.raises(AssertionError):
        shuffle_weight_bytes(b[:, :200])
    # the scale plane: the 8 bytes of row 16 nb + n, step s at (nb * steps + s) * 128 + 8 n
    K = 768
    mx = rng.integers(0, 256, (N, K // 32)).astype(np.uint8)
    ss = shuffle_scales_e8m0(mx)
    sflat, ssteps = ss.reshape(-1), K // 256
    for (nb, st, n) in ((0, 0, 0), (2, 2, 15), (1, 1, 6)):
        at = (nb * ssteps + st) * 128 + 8 * n
        assert np.array_equal(sflat[at:at + 8], mx[16 * nb + n, st * 8:][:8])
    assert np.array_equal(unshuffle_scales_e8m0(ss), mx)
    out = np.empty_like(mx)
    _capi.check(_capi.load().astergemm_shuffle_scales_e8m0(mx.ctypes.data, out.ctypes.data, N, K))
    assert np.array_equal(out, ss)
    assert _capi.load().astergemm_shuffle_scales_e8m0(mx.ctypes.data, out.ctypes.data, N, K + 32) != 0


def test_shuffle_scales_e8m0_lanes_is_what_a_lane_of_the_stream_kernel_loads():
    # lane 16 q + i of a wave loads the 8 bytes at 8 (16 q + i) of the 512 bytes of (64-row group
    # nb4, step s): byte 2 t + h is the scale of block 4 h + q of row 64 nb4 + 16 t + i, i.e. of
    # the 32 K-elements that lane feeds into MFMA h of that step for its row in tile t; the C-ABI
    # function writes the same bytes; the inverse restores the plane
    from aster_amd import _capi
    from aster_amd.kittens_helpers import shuffle_scales_e8m0_lanes, unshuffle_scales_e8m0_lanes
    rng = np.random.default_rng(6)
    N, K = 192, 768
    mx = rng.integers(0, 256, (N, K // 32)).astype(np.uint8)
    sh = shuffle_scales_e8m0_lanes(mx)
    flat, steps = sh.reshape(-1), K // 256
    for nb4 in range(N // 64):
        for st in range(steps):
            for lane in range(64):
                q, i = lane // 16, lane % 16
                got = flat[((nb4 * steps + st) * 64 + lane) * 8:][:8].reshape(4, 2)   # [t][h]
                want = mx[64 * nb4 + 16 * np.arange(4) + i][:, st * 8 + 4 * np.arange(2) + q]
                assert np.array_equal(got, want)
    assert np.array_equal(unshuffle_scales_e8m0_lanes(sh), mx)
    out = np.empty_like(mx)
    lib = _capi.load()
    _capi.check(lib.astergemm_shuffle_scales_e8m0_lanes(mx.ctypes.data, out.ctypes.data, N, K))
    assert np.array_equal(out, sh)
    assert lib.astergemm_shuffle_scales_e8m0_lanes(mx.ctypes.data, out.ctypes.data, N - 16, K) != 0
    assert lib.astergemm_shuffle_scales_e8m0_lanes(mx.ctypes.data, out.ctypes.data, N, K + 32) != 0
    with pytest.raises(AssertionError):
        shuffle_scales_e8m0_lanes(mx[:48])


def test_shuffle_scales_e8m0_lanes128_is_what_a_lane_of_the_stream_kernel_loads():
    # activations: groups of 128 rows (padded with the byte 127), per group and step one KiB in
    # which lane L = 16 q + i finds at byte 16 L + 2 t + h the scale of block 4 h + q of row
    # 128 g + 16 t + i (gemm_stream4db_kernel.hpp, A scales in lane order)
    from aster_amd import _capi
    from aster_amd.kittens_helpers import (mx_lanes128_bytes, shuffle_scales_e8m0_lanes128,
                                           unshuffle_scales_e8m0_lanes128)
    M, K = 328, 1024           # two whole groups and 72 rows of a third
    rng = np.random.default_rng(3)
    mx = rng.integers(0, 255, (M, K // 32), dtype=np.uint8)
    sh = shuffle_scales_e8m0_lanes128(mx)
    assert sh.shape == (mx_lanes128_bytes(M, K),) and mx_lanes128_bytes(M, K) == 3 * 4 * 1024
    steps = K // 256
    for g, s_, L, t, h in [(0, 0, 0, 0, 0), (1, 2, 37, 5, 1), (2, 3, 63, 7, 1), (2, 1, 8, 4, 0), (2, 0, 9, 4, 0)]:
        q, i = L // 16, L % 16
        row = 128 * g + 16 * t + i
        want = mx[row, 8 * s_ + 4 * h + q] if row < M else 127
        assert sh[(g * steps + s_) * 1024 + 16 * L + 2 * t + h] == want
    assert np.array_equal(unshuffle_scales_e8m0_lanes128(sh, M, K), mx)
    lib = _capi.load()
    out = np.zeros_like(sh)
    assert lib.astergemm_mx_lanes128_bytes(M, K) == sh.size
    _capi.check(lib.astergemm_shuffle_scales_e8m0_lanes128(mx.ctypes.data, out.ctypes.data, M, K))
    assert np.array_equal(out, sh)
    assert lib.astergemm_shuffle_scales_e8m0_lanes128(mx.ctypes.data, out.ctypes.data, M, K + 32) != 0
    with pytest.raises(AssertionError):
        shuffle_scales_e8m0_lanes128(mx[:, :-1])
