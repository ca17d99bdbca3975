"""Pins the oracle's number formats against fixtures the reference holds, torch's
independent converters, and brute force."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import formats as F


@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "kat.json")) as f:
        return json.load(f)


def test_e4m3_reference_code_points(kat):
    table = F.e4m3_decode_table()
    for code, value in kat["e4m3_codes"].items():
        assert table[int(code, 16)] == value
        assert F.e4m3_encode(np.array([value], np.float32))[0] == int(code, 16)
        assert F.e4m3_encode(np.array([-value], np.float32))[0] == int(code, 16) | 0x80


def test_e8m0_reference_code_points(kat):
    for code, value in kat["e8m0_codes"].items():
        assert F.e8m0_decode(np.array([int(code, 16)], np.uint8))[0] == value
    assert np.isnan(F.e8m0_decode(np.array([0xFF], np.uint8))[0])
    assert F.e8m0_decode(np.array([0], np.uint8))[0] == np.float32(2.0 ** -127)


def test_e4m3_decode_matches_torch():
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = F.e4m3_decode(codes)
    assert np.array_equal(np.isnan(want), np.isnan(got))
    ok = ~np.isnan(want)
    assert np.array_equal(want[ok].view(np.uint32), got[ok].view(np.uint32))


def test_e4m3_roundtrip_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    vals = F.e4m3_decode(codes)
    finite = ~np.isnan(vals)
    assert np.array_equal(F.e4m3_encode(vals)[finite], codes[finite])
    assert set(F.e4m3_encode(vals)[~finite].tolist()) <= {0x7F, 0xFF}


def test_e4m3_encode_matches_torch_in_range():
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(300000) * np.exp(rng.uniform(-14, 6, 300000))).astype(np.float32)
    x = x[np.abs(x) <= 448.0]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(F.e4m3_encode(x), want)


def test_e4m3_encode_matches_bit_level_scalar():
    rng = np.random.default_rng(8)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-16, 8, 20000))).astype(np.float32)
    # every midpoint between adjacent codes and both neighbours of it
    t = F.e4m3_decode_table()[:0x7F].astype(np.float64)
    mids = ((t[:-1] + t[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                        -mids, np.array([0.0, -0.0, 448, 449, 464, 465, 1e9, -1e9, np.inf, -np.inf,
                                         np.nan, 2.0 ** -10, 2.0 ** -9, 1e-30], np.float32)])
    vec = F.e4m3_encode(x)
    sca = np.array([F.e4m3_encode_scalar(v) for v in x], dtype=np.uint8)
    assert np.array_equal(vec, sca)


def test_e4m3_reference_inputs_of_cvt_pk_test():
    # The reference's converter test feeds float(i) and float(i) * 0.5, i = 0..63
    # (test/integration/test_conversion_pack_e2e.py:494-501): all in the normal
    # range, where the reference helper, RNE and torch agree.
    x = np.concatenate([np.arange(64, dtype=np.float32), np.arange(64, dtype=np.float32) * 0.5])
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(F.e4m3_encode(x), want)
    assert np.array_equal(F.e4m3_encode(x, subnormal="reference"), want)


def test_e4m3_saturation_and_specials():
    x = np.array([448.0, 449.0, 1e6, -1e6, np.inf, -np.inf, np.nan, 0.0, -0.0], np.float32)
    assert F.e4m3_encode(x).tolist() == [0x7E, 0x7E, 0x7E, 0xFE, 0x7F, 0xFF, 0x7F, 0x00, 0x80]


def test_e4m3_reference_helper_subnormal_mode_differs_only_below_min_normal():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(100000) * np.exp(rng.uniform(-14, 6, 100000))).astype(np.float32)
    a, b = F.e4m3_encode(x), F.e4m3_encode(x, subnormal="reference")
    diff = a != b
    assert np.all(np.abs(x[diff]) < 2.0 ** -6)
    # documented quirks of the helper (test_conversion_pack_e2e.py:132-143)
    q = np.array([5 * 2.0 ** -10, 1.5 * 2.0 ** -10, 7.5 * 2.0 ** -9], np.float32)
    assert F.e4m3_encode(q).tolist() == [2, 1, 8]
    assert F.e4m3_encode(q, subnormal="reference").tolist() == [3, 0, 7]


def test_bf16_matches_torch():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(200000) * np.exp(rng.uniform(-40, 40, 200000))).astype(np.float32)
    x = np.concatenate([x, np.array([0.0, -0.0, np.inf, -np.inf, 1.0, 1.00390625, 1.01171875,
                                     3.3895314e38, 1e-45], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = F.f32_to_bf16_bits(x)
    assert np.array_equal(got, want)
    assert np.array_equal(F.bf16_bits_to_f32(got).view(np.uint32), got.astype(np.uint32) << 16)
    nan = F.f32_to_bf16_bits(np.array([np.nan], np.float32))
    assert np.isnan(F.bf16_bits_to_f32(nan))[0]


def test_bf16_ties_to_even():
    # 1 + 2^-8 is halfway between 1.0 (even) and 1 + 2^-7; 1 + 3*2^-8 rounds up to even
    x = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8], np.float32)
    assert F.f32_to_bf16_bits(x).tolist() == [0x3F80, 0x3F82]


def test_e2m1_all_codes_roundtrip_and_ties():
    codes = np.arange(16, dtype=np.uint8)
    vals = F.e2m1_decode(codes)
    assert vals[:8].tolist() == [0, .5, 1, 1.5, 2, 3, 4, 6]
    assert np.array_equal(F.e2m1_encode(vals), codes)
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, 100.0, -5.0], np.float32)
    assert F.e2m1_decode(F.e2m1_encode(ties)).tolist() == [0, 1, 1, 2, 2, 4, 4, 6, 6, -4]


def test_e2m1_encode_is_nearest_by_brute_force():
    rng = np.random.default_rng(2)
    x = rng.uniform(-7, 7, 20000).astype(np.float32)
    grid = F.e2m1_decode(np.arange(16, dtype=np.uint8)).astype(np.float64)
    got = F.e2m1_decode(F.e2m1_encode(x)).astype(np.float64)
    best = np.min(np.abs(x.astype(np.float64)[:, None] - grid[None, :]), axis=1)
    assert np.array_equal(np.abs(got - x), best)


def test_nibble_packing_low_first():
    c = np.array([[1, 2, 3, 15]], np.uint8)
    p = F.pack_nibbles(c)
    assert p.tolist() == [[0x21, 0xF3]]
    assert np.array_equal(F.unpack_nibbles(p), c)


def test_mx_quantizer_closed_form():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((8, 128)) * np.exp(rng.uniform(-6, 6, (8, 1)))).astype(np.float32)
    packed, scales = F.quantize_mxfp4(x)
    assert packed.shape == (8, 64) and scales.shape == (8, 4)
    blk = x.reshape(8, 4, 32)
    amax = np.abs(blk).max(-1)
    want = np.floor(np.log2(amax.astype(np.float64))).astype(int) - 2 + 127
    assert np.array_equal(scales.astype(int), want)
    # scaled block maximum lands in [4, 8): it quantises to 4 or saturates at 6
    q = F.e2m1_decode(F.unpack_nibbles(packed)).reshape(8, 4, 32)
    assert np.all(np.abs(q).max(-1) >= 4.0)
    deq = F.dequantize_mxfp4(packed, scales)
    # error bound: half a grid step (<= 1 in scaled units, 2 where saturating 6..8)
    step = np.repeat(F.e8m0_decode(scales), 32, axis=-1)
    assert np.all(np.abs(deq - x) <= 2.0 * step + 1e-30)


def test_mx_quantizer_exact_on_representable_blocks():
    rng = np.random.default_rng(4)
    codes = rng.integers(0, 16, (4, 64)).astype(np.uint8)
    codes[:, 0::32] = 7  # make 6.0 the block maximum so the shared exponent is fixed
    sc = np.array([[120, 131], [127, 100], [1, 250], [127, 127]], np.uint8)
    x = F.dequantize_mxfp4(F.pack_nibbles(codes), sc)
    p2, s2 = F.quantize_mxfp4(x)
    assert np.array_equal(s2, sc)
    # -0 and +0 nibbles both decode to zero; compare values
    assert np.array_equal(F.dequantize_mxfp4(p2, s2), x)


def test_mx_quantizer_zero_and_nonfinite_blocks():
    x = np.zeros((1, 64), np.float32)
    x[0, 40] = np.inf
    p, s = F.quantize_mxfp4(x)
    assert s.tolist() == [[127, 0xFF]]
    assert np.all(p[0, :16] == 0)


def test_fp8_tensor_quantizer():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((64, 64)).astype(np.float32)
    q, s = F.quantize_fp8_tensor(x)
    assert s.dtype == np.float32 and s == np.float32(np.abs(x).max() / np.float32(448.0))
    assert np.abs(F.e4m3_decode(q)).max() == 448.0
    assert np.array_equal(q, F.e4m3_encode((x / s).astype(np.float32)))
    q0, s0 = F.quantize_fp8_tensor(np.zeros((4, 4), np.float32))
    assert s0 == 1.0 and not q0.any()
