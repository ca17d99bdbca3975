"""Runtime seam on the GPU: buffers, events, memory manager, and `execute_hsaco`
on the code object built from the same kernels (contracts of the reference's
test/integration/test_execution_core.py:198-500)."""
import os

import numpy as np
import pytest

from aster_amd import build as B
from aster_amd.execution import (FlushLLC, GpuBuffer, GpuEvent, GpuStream, InOutArray, InputArray,
                                 MemoryManager, OutputArray, execute_hsaco, system_has_gpu)
from oracle import gemm as G

pytestmark = pytest.mark.gpu


def test_system_has_gpu(gpu):
    assert system_has_gpu("gfx950") and not system_has_gpu("gfx942")


def test_gpu_buffer_roundtrip_and_contracts(gpu):
    for dt in (np.float32, np.float16, np.int32, np.uint8, np.float64):
        x = (np.arange(1000) % 251).astype(dt)
        buf = GpuBuffer(x.nbytes)
        buf.copy_from_host(x)
        y = np.zeros_like(x)
        buf.copy_to_host(y)
        assert np.array_equal(x, y)
        buf.free()
        buf.free()  # idempotent
    buf = GpuBuffer(16)
    assert buf.size_bytes == 16 and buf.ptr_value
    with pytest.raises(TypeError):
        buf.copy_from_host([1, 2, 3])
    with pytest.raises(TypeError):
        buf.copy_to_host("x")
    with pytest.raises(ValueError):
        buf.copy_from_host(np.zeros(100, np.float32))
    with pytest.raises(ValueError):
        buf.copy_to_host(np.zeros(100, np.float32))


def test_events_and_streams(gpu):
    s = GpuStream()
    s.synchronize()
    s.destroy()
    s.destroy()
    e0, e1 = GpuEvent(), GpuEvent()
    e0.record()
    e1.record()
    e1.synchronize()
    assert e1.elapsed_ms(e0) >= 0.0
    ns = e1.elapsed_ns(e0)
    assert isinstance(ns, int) and ns >= 0
    e0.destroy()
    e0.destroy()


def test_memory_manager_contracts(gpu):
    mm = MemoryManager()
    a = np.arange(64, dtype=np.float32)
    b = np.zeros(64, dtype=np.float32)
    buf = mm.register(a)
    assert isinstance(buf, GpuBuffer) and mm.register(a) is buf
    with pytest.raises(TypeError):
        mm.register([1, 2])
    mm.register(b, upload=False)
    assert mm.get_buffer(b) is not buf
    a[:] = 5
    mm.sync_to_gpu(a)
    a[:] = 0
    mm.sync_from_gpu(a)
    assert np.all(a == 5)
    other = np.zeros(4, np.float32)
    for fn in (mm.get_buffer, mm.sync_to_gpu, mm.sync_from_gpu, mm.release):
        with pytest.raises(KeyError):
            fn(other)
    mm.release(a)
    with pytest.raises(KeyError):
        mm.get_buffer(a)
    mm.release_all()
    mm.release_all()
    with pytest.raises(KeyError):
        mm.get_buffer(b)


def test_execute_hsaco_runs_the_code_object(gpu):
    assert os.path.exists(B.HSACO_PATH), "run python -m aster_amd.build"
    M, N, K = 160, 96, 72
    np.random.seed(42 + M + N + K)
    a = (np.random.randn(M, K) * 0.1).astype(np.float16)
    b = (np.random.randn(N, K) * 0.1).astype(np.float16)
    c = np.zeros(M * N, dtype=np.float32)
    seen = []
    grid = ((M + 127) // 128) * ((N + 127) // 128)
    times = execute_hsaco(B.HSACO_PATH, "gemm_cdna4",
                          [InputArray(a.flatten()), InputArray(b.flatten()), OutputArray(c), M, N, K],
                          grid_dim=(grid, 1, 1), block_dim=(256, 1, 1), num_iterations=3,
                          shared_bytes=65536, verify_fn=lambda args: seen.append(len(args)),
                          flush_llc=FlushLLC(1 << 20))
    assert len(times) == 3 and all(isinstance(t, int) and t > 0 for t in times)
    assert seen == [6]
    expected = (a.astype(np.float32) @ b.astype(np.float32).T).flatten()
    np.testing.assert_allclose(c, expected, rtol=1e-2, atol=1e-2)
    assert G.rel_l2(c, expected) <= 1e-3


def test_execute_hsaco_inout_and_missing_kernel(gpu):
    M = N = K = 128
    a = np.full((M, K), 0x3F80, np.uint16)
    c = np.zeros((M, N), dtype=np.uint16)
    execute_hsaco(B.HSACO_PATH, "gemm_cdna4_bf16", [InputArray(a), InputArray(a), c, M, N, K],
                  grid_dim=(1, 1, 1), block_dim=(256, 1, 1), shared_bytes=65536)
    assert np.all(c == 0x4300)  # 128.0 in bf16
    with pytest.raises(RuntimeError):
        execute_hsaco(B.HSACO_PATH, "no_such_kernel", [InOutArray(c)])


def test_failed_runtime_call_does_not_poison_later_launches(gpu):
    """A HIP call that failed (a kernel name the code object does not hold) leaves its error as
    the thread's last error; GEMM launches and quantiser calls that follow must not report it."""
    from aster_amd import gemm, quantize

    with pytest.raises(RuntimeError):
        execute_hsaco(B.HSACO_PATH, "no_such_kernel", [InOutArray(np.zeros(4, np.float32))])
    M, N, K = 16, 64, 4096
    a = np.full((M, K), 0x3F80, np.uint16)
    bufs = [GpuBuffer(M * K * 2), GpuBuffer(N * K * 2), GpuBuffer(M * N * 4)]
    bufs[0].copy_from_host(a)
    bufs[1].copy_from_host(np.full((N, K), 0x3F80, np.uint16))
    gemm.GemmPlan.create(M, N, K, "bf16", "f32").run(*(b.ptr_value for b in bufs))
    out = np.empty((M, N), np.float32)
    bufs[2].copy_to_host(out)
    assert np.all(out == K)
    with pytest.raises(RuntimeError):
        execute_hsaco(B.HSACO_PATH, "no_such_kernel", [InOutArray(np.zeros(4, np.float32))])
    q, s = quantize.quantize_fp8_tensor(np.linspace(-448, 448, 1024, dtype=np.float32))
    assert s == 1.0 and q[0] == 0xFE and q[-1] == 0x7E


def test_diag_mfma_rate_depends_on_operand_values(gpu):
    """Independent MFMAs over registers: zeros run near the published peak, random bf16 data
    well below it (the board's power limit), and both are plausible rates for this chip."""
    from aster_amd import _capi, gemm as AG
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(1 << 18) * 0.02).astype(np.float32)
    bits = (x.view(np.uint32) >> 16).astype(np.uint16)
    buf = GpuBuffer(bits.nbytes)
    buf.copy_from_host(bits)
    random_tf = AG.mfma_rate(buf.ptr_value, bits.nbytes, "bf16", target_ms=100)
    buf.copy_from_host(np.zeros_like(bits))
    zeros_tf = AG.mfma_rate(buf.ptr_value, bits.nbytes, "bf16", target_ms=100)
    fp8_tf = AG.mfma_rate(buf.ptr_value, bits.nbytes, "fp8_e4m3", target_ms=50)
    fp4_tf = AG.mfma_rate(buf.ptr_value, bits.nbytes, "mxfp4", target_ms=50)
    buf.free()
    assert 500.0 < random_tf < zeros_tf <= 2600.0
    assert zeros_tf < fp8_tf <= 5200.0 and fp8_tf < fp4_tf <= 10500.0
    with pytest.raises(_capi.AsterGemmError):
        AG.mfma_rate(0, 4096, "bf16")
    with pytest.raises(_capi.AsterGemmError):
        AG.mfma_rate(1 << 20, 100, "bf16")
