"""Pins the GEMM oracle: brute force, float64 BLAS, the C restatement, and the
closed-form known answers of the reference's MFMA tests."""
import json
import os

import numpy as np
import pytest

from oracle import cgemm, formats as F, gemm as G


@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "kat.json")) as f:
        return {c["name"]: c for c in json.load(f)["cases"]}


def _inputs(M, N, K, seed, scale=0.1, dtype=np.float16):
    # the reference's test inputs: seed 42 + M + N + K, randn * 0.1 -> f16
    # (contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:474-476)
    np.random.seed(seed)
    a = (np.random.randn(M, K) * scale).astype(dtype)
    b = (np.random.randn(N, K) * scale).astype(dtype)
    return a, b


@pytest.mark.parametrize("shape", [(3, 5, 7), (16, 16, 32), (17, 9, 40)])
def test_blas_oracle_matches_bruteforce(shape):
    M, N, K = shape
    a, b = _inputs(M, N, K, 42 + M + N + K)
    bf = G.gemm_bruteforce(a, b)
    assert G.rel_l2(G.gemm_f32(a, b), bf) < 1e-6
    assert G.rel_l2(G.gemm_f64(a, b), bf) < 1e-6
    assert G.rel_l2(cgemm.gemm_f32(a.astype(np.float32), b.astype(np.float32)), bf) < 1e-6


def test_oracle_detects_plausible_mistakes():
    a, b = _inputs(8, 8, 8, 1)
    good = G.gemm_bruteforce(a, b)
    assert G.rel_l2(a.astype(np.float32) @ b.astype(np.float32), good) > 0.5      # missing transpose
    assert G.rel_l2(G.gemm_f32(b, a), good) > 0.5                                  # swapped operands
    assert G.rel_l2(G.gemm_f32(a[:, :-1], b[:, :-1]), good) > 1e-3                 # dropped K term
    assert G.rel_l2(G.gemm_f32(a, -b), good) > 1.0                                  # wrong sign


@pytest.mark.parametrize("dtype_id,np_dt", [(G.F16, np.float16), (G.BF16, None), (G.FP8_E4M3, None),
                                             (G.MXFP4, None)])
def test_c_restatement_matches_numpy_on_raw_storage(dtype_id, np_dt):
    rng = np.random.default_rng(11)
    M, N, K = 37, 29, 96
    xa = rng.standard_normal((M, K)).astype(np.float32)
    xb = rng.standard_normal((N, K)).astype(np.float32)
    mx_a = mx_b = None
    if dtype_id == G.F16:
        ra, rb = xa.astype(np.float16), xb.astype(np.float16)
    elif dtype_id == G.BF16:
        ra, rb = F.f32_to_bf16_bits(xa), F.f32_to_bf16_bits(xb)
    elif dtype_id == G.FP8_E4M3:
        ra, rb = F.e4m3_encode(xa), F.e4m3_encode(xb)
    else:
        ra, mx_a = F.quantize_mxfp4(xa)
        rb, mx_b = F.quantize_mxfp4(xb)
    want = G.gemm_f32(G.decode_operand(ra, dtype_id, mx_a), G.decode_operand(rb, dtype_id, mx_b))
    got = cgemm.gemm_raw(ra, rb, dtype_id, M, N, K, mx_a, mx_b)
    assert G.rel_l2(got, want) < 1e-6


def test_kat_bf16_all_ones(kat):
    for name in ("bf16_16x16x32_all_ones", "bf16_32x32x16_all_ones"):
        c = kat[name]
        k = c["k"]
        a = np.full((16, k), int(c["a_bits"], 16), np.uint16)
        out = G.gemm(a, a, G.BF16, G.F32)
        assert np.all(out == c["expected"])


def test_kat_fp8_scaled(kat):
    c = kat["fp8_scaled_nonidentity"]
    a = np.full((16, c["k"]), int(c["a_byte"], 16), np.uint8)
    b = np.full((16, c["k"]), int(c["b_byte"], 16), np.uint8)
    sa = F.e8m0_decode(np.array([int(c["scale_a_e8m0"], 16)], np.uint8))[0]
    sb = F.e8m0_decode(np.array([int(c["scale_b_e8m0"], 16)], np.uint8))[0]
    assert (sa, sb) == (c["scale_a"], c["scale_b"])
    assert np.all(G.gemm_fp8(a, b, sa, sb, out_dtype=G.F32) == c["expected"])
    # identity scales would give 280 (the failure mode that test guards against)
    assert np.all(G.gemm_fp8(a, b, 1.0, 1.0, out_dtype=G.F32) == 280.0)


def test_kat_fp8_split_k_accumulate(kat):
    c = kat["fp8_split_k_accum"]
    k = c["k"]
    a = np.empty((16, k), np.uint8)
    b = np.empty((16, k), np.uint8)
    a[:, : k // 2], a[:, k // 2:] = (int(v, 16) for v in c["a_bytes_halves"])
    b[:, : k // 2], b[:, k // 2:] = (int(v, 16) for v in c["b_bytes_halves"])
    bias = np.full(16, c["c_init"], np.float32)
    out = G.gemm_fp8(a, b, 1.0, 1.0, out_dtype=G.F32, bias=bias)
    assert np.all(out == c["expected"])


def test_epilogue_order_and_casts():
    acc = np.array([[1.0, 2.0], [3.0, 4.0]], np.float32)
    bias = np.array([0.5, -0.5], np.float32)
    out = G.gemm_epilogue(acc, G.F32, 2.0, 0.25, bias)
    assert np.array_equal(out, np.array([[1.0, 0.5], [2.0, 1.5]], np.float32))
    bf = G.gemm_epilogue(np.array([[1.00390625]], np.float32), G.BF16)
    assert bf.dtype == np.uint16 and bf[0, 0] == 0x3F80
    h = G.gemm_epilogue(np.array([[65504.0]], np.float32), G.F16)
    assert h.view(np.float16)[0, 0] == np.float16(65504.0)


def test_mxfp4_gemm_linearity_in_block_scales():
    # Doubling one operand's e8m0 bytes doubles the product exactly.
    rng = np.random.default_rng(12)
    a = rng.integers(0, 256, (8, 64)).astype(np.uint8)
    b = rng.integers(0, 256, (8, 64)).astype(np.uint8)
    sa = rng.integers(120, 130, (8, 4)).astype(np.uint8)
    sb = rng.integers(120, 130, (8, 4)).astype(np.uint8)
    c1 = G.gemm_mxfp4(a, sa, b, sb, out_dtype=G.F32)
    c2 = G.gemm_mxfp4(a, sa + 1, b, sb, out_dtype=G.F32)
    assert np.array_equal(c2, 2 * c1)
