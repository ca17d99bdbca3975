"""Number formats of the GEMM path, as numpy bit arithmetic.  Test infrastructure.

bf16, OCP e4m3, OCP e2m1, e8m0, and the two quantisers (per-tensor fp8,
OCP-MX fp4 blocks).  Every encoder is round-to-nearest-even unless said
otherwise.
"""

from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------- bf16


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (uint16 bit patterns), round-to-nearest-even, NaN kept quiet."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# --------------------------------------------------------------------------- e4m3 (OCP)
# 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; S.1111.111 is NaN;
# largest finite 0x7E = 448.  gfx950 uses this flavour
# (reference: test/integration/test_conversion_pack_e2e.py:79-88, `_TARGET_IS_FNUZ`).


def e4m3_decode_table() -> np.ndarray:
    """float32[256]: value of every OCP e4m3 code."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 7
        if e == 0xF and m == 7:
            v = float("nan")
        elif e == 0:
            v = s * m * 2.0 ** -9
        else:
            v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[code] = v
    return out


_E4M3_TABLE = e4m3_decode_table()
_E4M3_POS = _E4M3_TABLE[:0x7F].astype(np.float64)  # codes 0x00..0x7E ascending
_E4M3_MIDS = (_E4M3_POS[:-1] + _E4M3_POS[1:]) / 2.0


def e4m3_decode(b: np.ndarray) -> np.ndarray:
    return _E4M3_TABLE[np.asarray(b, dtype=np.uint8)]


def e4m3_encode(x: np.ndarray, subnormal: str = "rne") -> np.ndarray:
    """fp32 -> OCP e4m3 bytes.

    Follows the reference converter `f32_to_fp8_e4m3(val, fnuz=False)`
    (test/integration/test_conversion_pack_e2e.py:91-167): round-to-nearest-even
    on the 3-bit mantissa with carry into the exponent, |x| > 448 saturates to
    0x7E, NaN and +-inf give S|0x7F, zero keeps its sign.

    `subnormal="rne"` (default) also rounds the subnormal range (|x| < 2^-6) to
    nearest-even, which is what `torch.float8_e4m3fn` and the hardware converter
    do.  `subnormal="reference"` reproduces the reference helper's behaviour
    there (:132-143): magnitudes below 2^-9 flush to zero, the rest round half
    up in units of 2^-9 and clamp to 7 units.
    """
    xf = np.ascontiguousarray(x, dtype=np.float32)
    bits = xf.view(np.uint32)
    sign = ((bits >> 31) & 1).astype(np.uint8) << 7
    mag = np.abs(xf).astype(np.float64)
    special = ~np.isfinite(xf)
    idx = np.searchsorted(_E4M3_MIDS, mag, side="left")  # mids strictly below |x|
    idx = np.minimum(idx, 0x7E)
    tie = (idx < 0x7E) & (mag == _E4M3_MIDS[np.minimum(idx, 0x7D)])
    idx = np.where(tie & (idx % 2 == 1), idx + 1, idx)
    idx = np.where(mag > 448.0, 0x7E, idx)
    if subnormal == "reference":
        sub = mag < 2.0 ** -6
        units = np.minimum(np.floor(mag * 512.0 + 0.5), 7.0)
        units = np.where(mag < 2.0 ** -9, 0.0, units)
        idx = np.where(sub, units.astype(np.int64), idx)
    elif subnormal != "rne":
        raise ValueError(subnormal)
    code = idx.astype(np.uint8) | sign
    code = np.where(special, sign | 0x7F, code)
    return code.astype(np.uint8)


def e4m3_encode_scalar(val: float) -> int:
    """Bit-level scalar encoder (RNE everywhere), independent of the table search
    above: used to pin `e4m3_encode` by brute force."""
    b = int(np.float32(val).view(np.uint32))
    s = (b >> 31) << 7
    e = (b >> 23) & 0xFF
    f = b & 0x7FFFFF
    if e == 0xFF:
        return s | 0x7F
    if e == 0 or e - 127 < -20:
        return s
    sig = (1 << 23) | f  # 1.f with 23 fraction bits
    exp = e - 127
    if exp >= -6:
        drop, base = 20, (exp + 7) << 3  # keep 3 fraction bits
    else:
        drop, base = 20 + (-6 - exp), 0  # subnormal: units of 2^-9
    q, rem = sig >> drop, sig & ((1 << drop) - 1)
    half = 1 << (drop - 1)
    if rem > half or (rem == half and (q & 1)):
        q += 1
    code = base + (q - 8 if exp >= -6 else q)  # mantissa carry flows into the exponent
    if code > 0x7E:
        code = 0x7E
    return s | code


# --------------------------------------------------------------------------- e2m1 / e8m0 (OCP MX)

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
_E2M1_MIDS = ((E2M1_VALUES[:-1] + E2M1_VALUES[1:]) / 2.0).astype(np.float64)


def e2m1_decode(code: np.ndarray) -> np.ndarray:
    c = np.asarray(code, dtype=np.uint8)
    v = E2M1_VALUES[c & 7]
    return np.where(c & 8, -v, v).astype(np.float32)


def e2m1_encode(x: np.ndarray) -> np.ndarray:
    """fp32 -> 4-bit e2m1 codes (uint8 in 0..15): RNE on the value grid, ties to
    the code with an even mantissa bit, |x| > 6 saturates, NaN -> sign|7."""
    xf = np.ascontiguousarray(x, dtype=np.float32)
    sign = ((xf.view(np.uint32) >> 31) & 1).astype(np.uint8) << 3
    mag = np.abs(xf).astype(np.float64)
    idx = np.searchsorted(_E2M1_MIDS, mag, side="left")
    idx = np.minimum(idx, 7)
    tie = (idx < 7) & (mag == _E2M1_MIDS[np.minimum(idx, 6)])
    idx = np.where(tie & (idx % 2 == 1), idx + 1, idx)
    idx = np.where(np.isnan(xf), 7, idx)
    return (idx.astype(np.uint8) | sign).astype(np.uint8)


def pack_nibbles(codes: np.ndarray) -> np.ndarray:
    """[.., K] 4-bit codes -> [.., K/2] bytes, element 2j in the low nibble."""
    c = np.asarray(codes, dtype=np.uint8)
    return (c[..., 0::2] | (c[..., 1::2] << 4)).astype(np.uint8)


def unpack_nibbles(packed: np.ndarray) -> np.ndarray:
    p = np.asarray(packed, dtype=np.uint8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = p & 0xF
    out[..., 1::2] = p >> 4
    return out


def e8m0_decode(b: np.ndarray) -> np.ndarray:
    """e8m0 scale byte -> fp32: 2^(byte-127); 0xFF is NaN.  The reference's
    scaled-MFMA test pins 0x7F=1, 0x80=2, 0x81=4
    (test/integration/mfma-f8f6f4-e2e.mlir:47-164)."""
    bb = np.asarray(b, dtype=np.uint8)
    v = np.ldexp(np.float64(1.0), bb.astype(np.int32) - 127)
    return np.where(bb == 0xFF, np.nan, v).astype(np.float32)


MX_BLOCK = 32


def quantize_mxfp4(x: np.ndarray):
    """OCP-MX v1.0 quantiser, blocks of 32 along the last axis.

    Returns (packed [.., K/2] uint8, scales [.., K/32] uint8).
    shared exponent = floor(log2(absmax)) - 2 (emax of e2m1), scale byte =
    clamp(shared + 127, 0, 254); a block holding NaN/inf gets 0xFF; an all-zero
    block gets byte 127 and zero nibbles (a choice: the spec leaves it open).
    Elements are RNE-saturated to e2m1 after division by 2^shared.
    """
    xf = np.ascontiguousarray(x, dtype=np.float32)
    K = xf.shape[-1]
    assert K % MX_BLOCK == 0
    blk = xf.reshape(xf.shape[:-1] + (K // MX_BLOCK, MX_BLOCK))
    amax = np.max(np.abs(blk), axis=-1)
    bad = ~np.isfinite(amax)
    _, e = np.frexp(np.where(bad | (amax == 0), 1.0, amax).astype(np.float64))
    shared = (e - 1) - 2
    shared = np.where(amax == 0, 0, shared)
    sbyte = np.clip(shared + 127, 0, 254).astype(np.int32)
    scale = np.ldexp(np.float64(1.0), sbyte - 127)
    q = e2m1_encode((blk.astype(np.float64) / scale[..., None]).astype(np.float32))
    sbyte = np.where(bad, 0xFF, sbyte).astype(np.uint8)
    return pack_nibbles(q.reshape(xf.shape)), sbyte


def dequantize_mxfp4(packed: np.ndarray, scales: np.ndarray) -> np.ndarray:
    v = e2m1_decode(unpack_nibbles(packed))
    s = np.repeat(e8m0_decode(scales), MX_BLOCK, axis=-1)
    return (v * s).astype(np.float32)


def quantize_fp8_tensor(x: np.ndarray):
    """Per-tensor absmax scaling: s = absmax/448 in fp32 (1.0 for an all-zero
    tensor), q = e4m3_rne_sat(fp32(x / s)).  Returns (bytes, np.float32 scale)."""
    xf = np.ascontiguousarray(x, dtype=np.float32)
    amax = np.float32(np.max(np.abs(xf))) if xf.size else np.float32(0)
    s = np.float32(amax / np.float32(448.0)) if amax > 0 else np.float32(1.0)
    return e4m3_encode((xf / s).astype(np.float32)), s
