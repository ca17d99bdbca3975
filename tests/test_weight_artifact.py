"""Weight artefact files: header layout, validation and checksums on the CPU (the C side is
host code); packing through the GPU quantisers and artefact -> GEMM end to end on the GPU."""
import ctypes
import struct
import zlib

import numpy as np
import pytest

from aster_amd import _capi, weights as W
from aster_amd.kittens_helpers import (shuffle_scales_e8m0, shuffle_scales_e8m0_lanes, shuffle_weight,
                                       shuffle_weight_bytes)


def _bf16(x):
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def test_header_is_128_bytes_with_the_documented_offsets():
    assert ctypes.sizeof(_capi.WeightHeader) == 128
    art = W.WeightArtifact.from_storage(np.arange(64 * 32, dtype=np.uint16).reshape(64, 32), "bf16",
                                        64, 32)
    raw = bytes(art.header)
    assert raw[:8] == b"ASTGEMW\0"
    version, hbytes, dtype, layout, scale_mode, tscale = struct.unpack_from("<IIIIIf", raw, 8)
    assert (version, hbytes, dtype, layout, scale_mode, tscale) == (1, 128, _capi.BF16, 0, 0, 1.0)
    n, k, poff, pbytes, soff, sbytes = struct.unpack_from("<qqqqqq", raw, 32)
    assert (n, k, poff, pbytes, soff, sbytes) == (64, 32, 256, 64 * 32 * 2, 0, 0)
    pcrc, scrc = struct.unpack_from("<II", raw, 80)
    assert pcrc == zlib.crc32(art.payload.tobytes()) and scrc == 0
    assert raw[88:] == b"\0" * 40


def test_crc32_is_the_zlib_polynomial():
    lib = _capi.load()
    for n in (0, 1, 9, 1000, 65537):
        buf = np.random.default_rng(n).integers(0, 256, n, dtype=np.uint8)
        assert lib.astergemm_weight_crc32(buf.ctypes.data, n) == zlib.crc32(buf.tobytes())
    check = np.frombuffer(b"123456789", dtype=np.uint8)
    assert lib.astergemm_weight_crc32(check.ctypes.data, 9) == 0xCBF43926   # the standard check value


@pytest.mark.parametrize("dtype,layout", [("bf16", "lds"), ("f16", "direct_b"), ("fp8_e4m3", "lds"),
                                           ("mxfp4", "lds"), ("fp8_e4m3", "direct_b"),
                                           ("mxfp4", "direct_b")])
def test_save_load_round_trip(tmp_path, dtype, layout):
    rng = np.random.default_rng(5)
    N, K = 48, 256
    scales, ts = None, 1.0
    if dtype in ("bf16", "f16"):
        bits = rng.integers(0, 1 << 16, (N, K), dtype=np.uint16)
    elif dtype == "fp8_e4m3":
        bits, ts = rng.integers(0, 256, (N, K), dtype=np.uint8), 0.0123
    else:
        bits = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        scales = rng.integers(100, 140, (N, K // 32), dtype=np.uint8)
    art = W.WeightArtifact.from_storage(bits, dtype, N, K, layout=layout, scales=scales,
                                        tensor_scale=ts)
    path = tmp_path / "w.astgemw"
    art.save(path)
    back = W.WeightArtifact.load(path)
    assert (back.dtype, back.layout, back.shape) == (dtype, layout, (N, K))
    assert np.array_equal(np.asarray(back.payload), bits.reshape(-1).view(np.uint8))
    assert back.tensor_scale == np.float32(ts)
    if scales is not None:
        assert np.array_equal(np.asarray(back.scales), scales.reshape(-1))
        assert back.header.scales_offset % 256 == 0
    raw = np.fromfile(path, dtype=np.uint8)
    assert _capi.load().astergemm_weight_verify(raw.ctypes.data, raw.size) == 0
    c = _capi.Config()
    _capi.check(_capi.load().astergemm_weight_config(ctypes.byref(back.header), 16, _capi.F32,
                                                    ctypes.byref(c)))
    assert (c.M, c.N, c.K, c.dtype_ab, c.dtype_c, c.operand_path) == (
        16, N, K, _capi.DTYPE_NAMES[dtype], _capi.F32, 1 if layout == "direct_b" else 0)
    assert c.scale_mode == {"bf16": 0, "f16": 0, "fp8_e4m3": 1, "mxfp4": 2}[dtype]


def test_corrupt_files_are_refused_with_a_reason(tmp_path):
    rng = np.random.default_rng(6)
    art = W.WeightArtifact.from_storage(rng.integers(0, 256, (32, 64), dtype=np.uint8), "mxfp4", 32,
                                        128, scales=rng.integers(0, 255, (32, 4), dtype=np.uint8))
    path = tmp_path / "w.astgemw"
    art.save(path)
    good = np.fromfile(path, dtype=np.uint8)
    lib = _capi.load()

    def refused(img, msg, fn=lib.astergemm_weight_verify):
        assert fn(img.ctypes.data, img.size) == -22
        assert msg in lib.astergemm_last_error().decode()

    bad = good.copy(); bad[0] ^= 1
    refused(bad, "bad magic")
    bad = good.copy(); bad[8] = 2
    refused(bad, "unsupported version")
    bad = good.copy(); bad[32] += 1                      # N no longer matches the section sizes
    refused(bad, "section sizes")
    bad = good.copy(); bad[300] ^= 0x10
    refused(bad, "payload checksum")
    bad = good.copy(); bad[-1] ^= 0x01
    refused(bad, "scale plane checksum")
    refused(good[:-8].copy(), "outside the file")
    refused(good[:100].copy(), "shorter than the header")
    # the Python loader raises the same errors
    bad = good.copy(); bad[300] ^= 0x10
    bad.tofile(tmp_path / "bad.astgemw")
    with pytest.raises(_capi.AsterGemmError, match="payload checksum"):
        W.WeightArtifact.load(tmp_path / "bad.astgemw")
    assert W.WeightArtifact.load(tmp_path / "bad.astgemw", verify=False).shape == (32, 128)


def test_packing_rules():
    with pytest.raises(_capi.AsterGemmError, match="128-byte steps"):
        W.WeightArtifact.from_storage(np.zeros((16, 32), np.uint8), "fp8_e4m3", 16, 32, layout="direct_b")
    with pytest.raises(_capi.AsterGemmError, match="128-byte steps"):
        W.WeightArtifact.from_storage(np.zeros((16, 64), np.uint8), "fp8_e4m3", 16, 64, layout="direct_b_k8")
    assert W.WeightArtifact.from_storage(np.zeros((16, 128), np.uint8), "fp8_e4m3", 16, 128,
                                         layout="direct_b_k8").shape == (16, 128)
    with pytest.raises(_capi.AsterGemmError, match="N % 16"):
        W.WeightArtifact.from_storage(np.zeros((8, 32), np.uint16), "bf16", 8, 32, layout="direct_b")
    with pytest.raises(ValueError, match="scale plane"):
        W.WeightArtifact.from_storage(np.zeros((16, 16), np.uint8), "mxfp4", 16, 32)
    with pytest.raises(ValueError, match="payload has"):
        W.WeightArtifact.from_storage(np.zeros((16, 31), np.uint16), "bf16", 16, 32)
    w = np.random.default_rng(1).standard_normal((32, 64)).astype(np.float32)
    plain = W.WeightArtifact.from_f32(w, "bf16")
    shuf = W.WeightArtifact.from_f32(w, "bf16", layout="direct_b")
    assert np.array_equal(plain.payload.view(np.uint16).reshape(32, 64), _bf16(w))
    assert np.array_equal(shuf.payload.view(np.uint16).reshape(32, 64), shuffle_weight(_bf16(w)))


# ---- GPU: pack with the device quantisers, save, load, multiply -------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("dtype,layout,M,N,K", [("bf16", "lds", 16, 512, 4096), ("bf16", "direct_b", 16, 512, 4096),
                                                ("bf16", "direct_b_k8", 264, 512, 1024),
                                                ("f16", "lds", 40, 264, 256), ("fp8_e4m3", "lds", 16, 512, 4096),
                                                ("fp8_e4m3", "lds", 300, 256, 512), ("mxfp4", "lds", 64, 256, 1024),
                                                ("fp8_e4m3", "direct_b", 16, 528, 4096),
                                                ("fp8_e4m3", "direct_b_k8", 264, 528, 1152),
                                                ("mxfp4", "direct_b", 9, 528, 8192),
                                                ("mxfp4", "direct_b_k8", 264, 576, 2048)])
def test_artifact_to_gemm_matches_the_oracle(tmp_path, dtype, layout, M, N, K):
    from aster_amd import quantize as Q
    from aster_amd.execution import GpuBuffer
    from oracle import formats as F, gemm as G

    rng = np.random.default_rng(77)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    print(f"artifact {dtype} {layout} M={M} N={N} K={K}", flush=True)
    W.WeightArtifact.from_f32(w, dtype, layout=layout).save(tmp_path / "w.astgemw")
    art = W.WeightArtifact.load(tmp_path / "w.astgemw")
    dev = art.to_device()
    out = np.empty((M, N), np.float32)
    d_out = GpuBuffer(out.nbytes)
    kw = {}
    if dtype in ("bf16", "f16"):
        xs = _bf16(x) if dtype == "bf16" else x.astype(np.float16)
        want = G.gemm(xs, _bf16(w) if dtype == "bf16" else w.astype(np.float16),
                      G.BF16 if dtype == "bf16" else G.F16, G.F32)
        bar = 1e-5
    elif dtype == "fp8_e4m3":
        xs, sx = F.quantize_fp8_tensor(x)
        wq, sw = F.quantize_fp8_tensor(w)
        stored = np.asarray(art.payload).reshape(N, K)
        assert np.array_equal(stored, wq if layout == "lds" else shuffle_weight_bytes(wq))
        assert art.tensor_scale == sw
        d_sx = GpuBuffer(4); d_sx.copy_from_host(np.array([sx], np.float32))
        kw["scale_x"] = d_sx.ptr_value
        want = G.gemm_fp8(xs, wq, sx, sw, out_dtype=G.F32)
        bar = 1e-4
    else:
        xs, mx = F.quantize_mxfp4(x)
        wq, ws = F.quantize_mxfp4(w)
        stored, plane = np.asarray(art.payload).reshape(N, K // 2), np.asarray(art.scales).reshape(N, K // 32)
        assert np.array_equal(stored, shuffle_weight_bytes(wq) if layout != "lds" else wq)
        assert np.array_equal(plane, {"lds": lambda s: s, "direct_b": shuffle_scales_e8m0,
                                      "direct_b_k8": shuffle_scales_e8m0_lanes}[layout](ws))
        d_mx = GpuBuffer(mx.nbytes); d_mx.copy_from_host(mx)
        kw["mx_x"] = d_mx.ptr_value
        want = G.gemm_mxfp4(xs, mx, wq, ws, out_dtype=G.F32)
        bar = 1e-5
    d_x = GpuBuffer(xs.nbytes); d_x.copy_from_host(np.ascontiguousarray(xs))
    dev.run(d_x.ptr_value, d_out.ptr_value, M, "f32", **kw)
    d_out.copy_to_host(out)
    if layout == "direct_b":
        assert dev.plan(M, "f32").info.name.decode().startswith("skinnyd")
    if layout == "direct_b_k8":
        assert dev.plan(M, "f32").info.name.decode().startswith("streamdb")
    assert G.rel_l2(out, G.output_to_f32(want, G.F32)) <= bar
    dev.free()
