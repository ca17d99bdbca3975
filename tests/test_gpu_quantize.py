"""GPU parity of the operand quantisers: bytes out of the HIP kernels (through the C-ABI)
must equal the oracle's, bit for bit: e4m3 codes and the fp32 tensor scale; e2m1 nibbles and
e8m0 block scale bytes.  The e4m3 oracle is itself pinned against the converter vectors of
the reference's tests (tests/test_oracle_formats.py)."""
import numpy as np
import pytest

from aster_amd import _capi, gemm as AG, quantize as Q
from aster_amd.execution import GpuBuffer
from oracle import formats as F, gemm as G

pytestmark = pytest.mark.gpu


def _special_f32():
    codes = F.e4m3_decode(np.arange(256, dtype=np.uint8)).astype(np.float32)
    fin = np.unique(codes[np.isfinite(codes)])
    mids = ((fin[:-1].astype(np.float64) + fin[1:]) / 2).astype(np.float32)
    up, dn = np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))
    return np.concatenate([fin, mids, up, dn]).astype(np.float32)


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 1023, 4096, 65537, 1 << 20])
def test_fp8_tensor_quantiser_matches_oracle(n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * rng.choice([1e-3, 0.05, 1.0, 40.0], n)).astype(np.float32)
    print(f"quantize_fp8_tensor n={n}", flush=True)
    q, s = Q.quantize_fp8_tensor(x)
    qo, so = F.quantize_fp8_tensor(x)
    assert np.float32(s).tobytes() == np.float32(so).tobytes()
    assert np.array_equal(q, qo)


def test_fp8_tensor_quantiser_rounding_cases():
    # absmax 448 -> scale exactly 1: every code, every midpoint between codes and both
    # neighbours of each midpoint go through the encoder unscaled
    sp = _special_f32()
    x = np.concatenate([sp, -sp, np.array([0.0, -0.0, 2.0 ** -10, 2.0 ** -11, 1.5 * 2.0 ** -10,
                                           1e-45, -1e-45, 1e-40], np.float32)])
    assert np.max(np.abs(x)) == 448.0
    print(f"quantize_fp8_tensor rounding cases n={x.size}", flush=True)
    q, s = Q.quantize_fp8_tensor(x)
    qo, so = F.quantize_fp8_tensor(x)
    assert s == 1.0 and so == 1.0
    assert np.array_equal(q, qo)
    # signed zeros and the tie at half the smallest subnormal
    assert q[x.size - 8] == 0x00 and q[x.size - 7] == 0x80 and q[x.size - 6] == 0x00


@pytest.mark.parametrize("case", ["zeros", "nan", "inf", "empty", "huge", "tiny"])
def test_fp8_tensor_quantiser_edge_tensors(case):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(1000).astype(np.float32)
    if case == "zeros":
        x[:] = 0
        x[3] = -0.0
    elif case == "nan":
        x[17] = np.nan
    elif case == "inf":
        x[99] = -np.inf
    elif case == "empty":
        x = x[:0]
    elif case == "huge":
        x *= np.float32(1e37)
    elif case == "tiny":
        x *= np.float32(1e-41)
    print(f"quantize_fp8_tensor edge {case}", flush=True)
    q, s = Q.quantize_fp8_tensor(x)
    with np.errstate(all="ignore"):
        qo, so = F.quantize_fp8_tensor(x)
    assert np.float32(s).tobytes() == np.float32(so).tobytes()
    assert np.array_equal(q, qo)


def test_absmax_matches_numpy():
    rng = np.random.default_rng(7)
    for n in (0, 1, 7, 1000, 300001):
        x = rng.standard_normal(n).astype(np.float32)
        if n > 5:
            x[n // 2] = -77.25
        src, out = GpuBuffer(max(x.nbytes, 16)), GpuBuffer(4)
        src.copy_from_host(x)
        print(f"absmax n={n}", flush=True)
        Q.absmax_device(src.ptr_value, n, out.ptr_value)
        got = np.empty(1, np.float32)
        out.copy_to_host(got)
        assert got[0] == (np.max(np.abs(x)) if n else 0.0)


def _mx_input(rows, K, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    # every block its own magnitude, over the whole fp32 exponent range
    e = rng.integers(-140, 126, size=(rows, K // 32))
    x = (x.astype(np.float64) * np.ldexp(1.0, np.repeat(e, 32, axis=1))).astype(np.float32)
    return x


@pytest.mark.parametrize("rows,K", [(1, 32), (3, 64), (16, 4096), (257, 1024), (64, 14336)])
def test_mxfp4_quantiser_matches_oracle(rows, K):
    x = _mx_input(rows, K, rows * 7 + K)
    print(f"quantize_mxfp4 rows={rows} K={K}", flush=True)
    p, s = Q.quantize_mxfp4(x)
    po, so = F.quantize_mxfp4(x)
    assert np.array_equal(s, so)
    assert np.array_equal(p, po)


def test_mxfp4_quantiser_special_blocks():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((8, 256)).astype(np.float32)
    x[0, 0:32] = 0.0                       # all-zero block -> scale byte 127, zero nibbles
    x[0, 5] = -0.0
    x[1, 32:64] = np.nan                   # NaN block -> 0xFF
    x[2, 64:96][3] = np.inf                # inf element -> 0xFF
    x[3, 0:32] *= np.float32(1e-44)        # fp32-subnormal block
    x[3, 32:64] = np.float32(2.0 ** -149)
    x[4, 0:32] *= np.float32(3e38)         # top of the fp32 range (may overflow to inf)
    x[4, 32:64] = np.float32(2.0 ** 127)
    # ties of the e2m1 grid with absmax 6 (scale 1): .25 .75 1.25 1.75 2.5 3.5 5 and neighbours
    t = np.array([6, .25, .75, 1.25, 1.75, 2.5, 3.5, 5, -.25, -.75, -1.25, -1.75, -2.5, -3.5, -5,
                  .5, 1, 1.5, 2, 3, 4, 0.2499999, 0.2500001, 5.0000005, 4.9999995, 0, -0.0,
                  7.9, 1e-30, -1e-30, 0.7499999, 0.7500001], np.float32)
    assert t.size == 32
    x[5, 0:32] = t
    x[5, 32:64] = t * np.float32(2.0 ** -20)
    x[6, 0:32] = 7.9999995                 # absmax just below 8 -> exponent 0, saturates to 6
    x[6, 32:64] = 8.0
    print("quantize_mxfp4 special blocks", flush=True)
    p, s = Q.quantize_mxfp4(x)
    with np.errstate(all="ignore"):
        po, so = F.quantize_mxfp4(x)
    assert np.array_equal(s, so)
    assert np.array_equal(p, po)
    assert s[0, 0] == 127 and p[0, 2] == 0x80 and not np.delete(p[0, :16], 2).any()
    assert s[1, 1] == 0xFF and s[2, 2] == 0xFF


def test_mxfp4_quantiser_strided_source_and_bad_arguments():
    rows, K, ld = 5, 96, 128
    x = _mx_input(rows, ld, 3)
    src, pk, sc = GpuBuffer(x.nbytes), GpuBuffer(rows * K // 2), GpuBuffer(rows * K // 32)
    src.copy_from_host(x)
    print("quantize_mxfp4 strided", flush=True)
    Q.quantize_mxfp4_device(src.ptr_value, rows, K, pk.ptr_value, sc.ptr_value, ld_src=ld)
    p, s = np.empty((rows, K // 2), np.uint8), np.empty((rows, K // 32), np.uint8)
    pk.copy_to_host(p)
    sc.copy_to_host(s)
    po, so = F.quantize_mxfp4(np.ascontiguousarray(x[:, :K]))
    assert np.array_equal(p, po) and np.array_equal(s, so)
    with pytest.raises(_capi.AsterGemmError, match="K % 32"):
        Q.quantize_mxfp4_device(src.ptr_value, rows, 48, pk.ptr_value, sc.ptr_value)
    with pytest.raises(_capi.AsterGemmError, match="ld_src"):
        Q.quantize_mxfp4_device(src.ptr_value, rows, K, pk.ptr_value, sc.ptr_value, ld_src=64)
    with pytest.raises(_capi.AsterGemmError, match="aligned"):
        Q.quantize_mxfp4_device(src.ptr_value + 4, rows, K, pk.ptr_value, sc.ptr_value)
    with pytest.raises(_capi.AsterGemmError, match="aligned"):
        Q.quantize_fp8_tensor_device(src.ptr_value + 4, 8, pk.ptr_value, sc.ptr_value)


def test_quantise_then_gemm_on_device_fp8():
    """fp32 operands in HBM -> device quantiser -> fp8 GEMM, nothing through the host; the
    result equals the oracle's GEMM on the oracle's quantised operands."""
    M, N, K = 256, 512, 1024
    rng = np.random.default_rng(21)
    xa = rng.standard_normal((M, K)).astype(np.float32)
    xb = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    fa, fb = GpuBuffer(xa.nbytes), GpuBuffer(xb.nbytes)
    qa, qb, sa, sb = GpuBuffer(M * K), GpuBuffer(N * K), GpuBuffer(4), GpuBuffer(4)
    dc = GpuBuffer(M * N * 2)
    fa.copy_from_host(xa)
    fb.copy_from_host(xb)
    print("quantise + gemm fp8", flush=True)
    Q.quantize_fp8_tensor_device(fa.ptr_value, M * K, qa.ptr_value, sa.ptr_value)
    Q.quantize_fp8_tensor_device(fb.ptr_value, N * K, qb.ptr_value, sb.ptr_value)
    plan = AG.GemmPlan.create(M, N, K, "fp8_e4m3", "bf16")
    plan.run(qa.ptr_value, qb.ptr_value, dc.ptr_value, scale_a=sa.ptr_value, scale_b=sb.ptr_value)
    out = np.empty((M, N), np.uint16)
    dc.copy_to_host(out)
    a_q, s_a = F.quantize_fp8_tensor(xa)
    b_q, s_b = F.quantize_fp8_tensor(xb)
    want = G.gemm_fp8(a_q, b_q, s_a, s_b, out_dtype=G.BF16)
    rel = G.rel_l2(G.output_to_f32(out, G.BF16), G.output_to_f32(want, G.BF16))
    assert rel <= 1e-3, rel
    # and the quantised GEMM stays near the fp32 product (e4m3 has 3 mantissa bits)
    assert G.rel_l2(G.output_to_f32(out, G.BF16), G.gemm_f32(xa, xb)) < 0.06


def test_quantise_then_gemm_on_device_mxfp4():
    M, N, K = 256, 256, 1024
    rng = np.random.default_rng(22)
    xa = rng.standard_normal((M, K)).astype(np.float32)
    xb = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    fa, fb = GpuBuffer(xa.nbytes), GpuBuffer(xb.nbytes)
    pa, pb = GpuBuffer(M * K // 2), GpuBuffer(N * K // 2)
    ma, mb = GpuBuffer(M * K // 32), GpuBuffer(N * K // 32)
    dc = GpuBuffer(M * N * 4)
    fa.copy_from_host(xa)
    fb.copy_from_host(xb)
    print("quantise + gemm mxfp4", flush=True)
    Q.quantize_mxfp4_device(fa.ptr_value, M, K, pa.ptr_value, ma.ptr_value)
    Q.quantize_mxfp4_device(fb.ptr_value, N, K, pb.ptr_value, mb.ptr_value)
    plan = AG.GemmPlan.create(M, N, K, "mxfp4", "f32")
    plan.run(pa.ptr_value, pb.ptr_value, dc.ptr_value, mx_a=ma.ptr_value, mx_b=mb.ptr_value)
    out = np.empty((M, N), np.float32)
    dc.copy_to_host(out)
    a_p, a_s = F.quantize_mxfp4(xa)
    b_p, b_s = F.quantize_mxfp4(xb)
    want = G.gemm_mxfp4(a_p, a_s, b_p, b_s, out_dtype=G.F32)
    rel = G.rel_l2(out, G.output_to_f32(want, G.F32))
    assert rel <= 1e-3, rel


@pytest.mark.parametrize("src", ["bf16", "f16"])
def test_quantisers_take_16_bit_sources(src):
    """bf16 / f16 sources (what a GEMM of this library writes) give the bytes of the widened
    values, bit for bit."""
    rng = np.random.default_rng(91)
    x32 = (rng.standard_normal((48, 4096)) * rng.choice([1e-3, 0.1, 1.0, 30.0], (48, 1))).astype(np.float32)
    if src == "bf16":
        bits = F.f32_to_bf16_bits(x32)
        wide = F.bf16_bits_to_f32(bits)
        host = bits
    else:
        host = x32.astype(np.float16)
        wide = host.astype(np.float32)
    host[0, :40] = 0                                   # an all-zero block and signed zeros
    wide[0, :40] = 0
    print(f"quantisers from {src}", flush=True)
    q, s = Q.quantize_fp8_tensor(host, src)
    qo, so = F.quantize_fp8_tensor(wide)
    assert np.float32(s).tobytes() == np.float32(so).tobytes() and np.array_equal(q, qo)
    p, sc = Q.quantize_mxfp4(host, src)
    po, sco = F.quantize_mxfp4(wide)
    assert np.array_equal(sc, sco) and np.array_equal(p, po)
    # odd lengths take the scalar tail
    q, s = Q.quantize_fp8_tensor(host.reshape(-1)[:1003], src)
    qo, so = F.quantize_fp8_tensor(wide.reshape(-1)[:1003])
    assert np.float32(s).tobytes() == np.float32(so).tobytes() and np.array_equal(q, qo)


def test_gemm_output_feeds_the_next_quantised_gemm():
    """bf16 GEMM -> MXFP4 quantiser on its bf16 output -> MXFP4 decode GEMM, all on the device."""
    M, K1, K2, N = 16, 1024, 4096, 512
    rng = np.random.default_rng(92)
    x = F.f32_to_bf16_bits(rng.standard_normal((M, K1)).astype(np.float32))
    w1 = F.f32_to_bf16_bits((rng.standard_normal((K2, K1)) * 0.03).astype(np.float32))
    w2 = (rng.standard_normal((N, K2)) * 0.05).astype(np.float32)
    w2p, w2s = F.quantize_mxfp4(w2)
    bufs = {k: GpuBuffer(v.nbytes) for k, v in dict(x=x, w1=w1, w2p=w2p, w2s=w2s).items()}
    for k, v in dict(x=x, w1=w1, w2p=w2p, w2s=w2s).items():
        bufs[k].copy_from_host(np.ascontiguousarray(v))
    h, hp, hs, y = GpuBuffer(M * K2 * 2), GpuBuffer(M * K2 // 2), GpuBuffer(M * K2 // 32), GpuBuffer(M * N * 4)
    print("bf16 gemm -> mxfp4 quantise -> mxfp4 gemm", flush=True)
    AG.GemmPlan.create(M, K2, K1, "bf16", "bf16").run(bufs["x"].ptr_value, bufs["w1"].ptr_value, h.ptr_value)
    Q.quantize_mxfp4_device(h.ptr_value, M, K2, hp.ptr_value, hs.ptr_value, src_dtype="bf16")
    plan = AG.GemmPlan.create(M, N, K2, "mxfp4", "f32")
    assert plan.info.name.decode().startswith("skinnyx_mxfp4")
    plan.run(hp.ptr_value, bufs["w2p"].ptr_value, y.ptr_value, mx_a=hs.ptr_value,
             mx_b=bufs["w2s"].ptr_value)
    out = np.empty((M, N), np.float32)
    y.copy_to_host(out)
    # oracle: the device's own bf16 intermediate, quantised and multiplied on the CPU
    hb = np.empty((M, K2), np.uint16)
    h.copy_to_host(hb)
    hq, hsc = F.quantize_mxfp4(F.bf16_bits_to_f32(hb))
    want = G.gemm_mxfp4(hq, hsc, w2p, w2s, out_dtype=G.F32)
    assert G.rel_l2(out, G.output_to_f32(want, G.F32)) <= 1e-5


@pytest.mark.parametrize("dtype_ab,path", [("bf16", "direct_b"), ("f16", "direct_b_k8"), ("fp8_e4m3", "direct_b"),
                                           ("fp8_e4m3", "direct_b_k8"), ("mxfp4", "direct_b"),
                                           ("mxfp4", "direct_b_k8")])
def test_preshuffle_on_the_device_writes_the_bytes_of_the_host_functions(gpu, dtype_ab, path):
    # the five pre-shuffled layouts, device to device, against kittens_helpers (which the C host
    # functions are tested against): same bytes; N, K with several row blocks and steps
    from aster_amd import kittens_helpers as H
    from aster_amd.execution import GpuBuffer
    N, K = 192, 1280
    rng = np.random.default_rng(8)
    mx = rng.integers(0, 256, (N, K // 32)).astype(np.uint8)
    if dtype_ab in ("bf16", "f16"):
        b = rng.integers(0, 65536, (N, K)).astype(np.uint16)
        want = (H.shuffle_weight if path == "direct_b" else H.shuffle_weight_k8)(b)
    else:
        b = rng.integers(0, 256, (N, K if dtype_ab == "fp8_e4m3" else K // 2)).astype(np.uint8)
        want = H.shuffle_weight_bytes(b)
    want_mx = (H.shuffle_scales_e8m0 if path == "direct_b" else H.shuffle_scales_e8m0_lanes)(mx)
    d_b, d_o, d_mx, d_mo = GpuBuffer(b.nbytes), GpuBuffer(b.nbytes), GpuBuffer(mx.nbytes), GpuBuffer(mx.nbytes)
    d_b.copy_from_host(b)
    d_mx.copy_from_host(mx)
    d_o.copy_from_host(np.zeros_like(b))
    d_mo.copy_from_host(np.zeros_like(mx))
    print(f"preshuffle {dtype_ab} {path}", flush=True)
    Q.preshuffle_device(d_b.ptr_value, d_o.ptr_value, N, K, dtype_ab, path,
                        d_mx_src=d_mx.ptr_value, d_mx_dst=d_mo.ptr_value)
    got, got_mx = np.zeros_like(b), np.zeros_like(mx)
    d_o.copy_to_host(got)
    d_mo.copy_to_host(got_mx)
    assert np.array_equal(got, want)
    if dtype_ab == "mxfp4":
        assert np.array_equal(got_mx, want_mx)
    else:
        assert not got_mx.any()     # no scale plane for these types: left alone
    with pytest.raises(_capi.AsterGemmError):   # in place is refused
        Q.preshuffle_device(d_b.ptr_value, d_b.ptr_value, N, K, dtype_ab, path,
                            d_mx_src=d_mx.ptr_value, d_mx_dst=d_mo.ptr_value)
    for bf in (d_b, d_o, d_mx, d_mo):
        bf.free()
