"""The entry point that allocates nothing (`astergemm_run_noalloc`) against `astergemm_run`.

Shapes whose rows are cut into K ranges keep their fp32 partial sums in a scratch array built
into the library instead of an allocated workspace; the results must be the same bits.  Two calls
in a row share the array, the second smaller than the first; a shape that needs no workspace and
one that needs more than the array holds are covered as well, and so is a HIP graph that holds
two launches of it and is replayed on fresh activations.
"""
import ctypes
import os

import numpy as np
import pytest

from aster_amd import _capi, gemm as AG
from aster_amd.execution import GpuBuffer
from oracle import formats as F, gemm as G

pytestmark = pytest.mark.gpu


def _bf16(rng, shape, std):
    return F.f32_to_bf16_bits((rng.standard_normal(shape) * std).astype(np.float32))


def _both_ways(M, N, K, seed):
    rng = np.random.default_rng(seed)
    a, b = _bf16(rng, (M, K), 1.0), _bf16(rng, (N, K), 0.02)
    plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16")
    bufs = [GpuBuffer(a.nbytes), GpuBuffer(b.nbytes), GpuBuffer(M * N * 2), GpuBuffer(M * N * 2)]
    bufs[0].copy_from_host(a)
    bufs[1].copy_from_host(b)
    outs = []
    for i, run in enumerate((plan.run, plan.run_noalloc)):
        out = np.full((M, N), 0x7FC1, np.uint16)
        bufs[2 + i].copy_from_host(out)
        print(f"{run.__name__} {plan.info.name.decode()} M={M} N={N} K={K} "
              f"workspace={plan.workspace_bytes()}", flush=True)
        run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2 + i].ptr_value)
        bufs[2 + i].copy_to_host(out)
        outs.append(out)
    for bf in bufs:
        bf.free()
    want = G.gemm(a, b, G.BF16, G.BF16)
    return plan, outs[0], outs[1], want


def test_noalloc_matches_run_on_two_calls_in_a_row(gpu):
    # split K on the 128 x 128 kernel: 8 K ranges x 128 x 4096 x 4 bytes = the whole 16 MiB array
    plan, ref, got, want = _both_ways(128, 4096, 14336, seed=7)
    assert plan.workspace_bytes() == _capi.NOALLOC_SCRATCH_BYTES
    assert np.array_equal(ref, got)
    assert G.rel_l2(F.bf16_bits_to_f32(got), F.bf16_bits_to_f32(want)) <= 1e-3
    # then a smaller one through the same array: a decode shape in K ranges
    plan, ref, got, want = _both_ways(16, 520, 14336, seed=8)
    assert 0 < plan.workspace_bytes() < _capi.NOALLOC_SCRATCH_BYTES
    assert np.array_equal(ref, got)
    assert G.rel_l2(F.bf16_bits_to_f32(got), F.bf16_bits_to_f32(want)) <= 1e-3
    # and a shape without K ranges: the array is not touched at all
    plan, ref, got, want = _both_ways(264, 520, 512, seed=9)
    assert plan.workspace_bytes() == 0
    assert np.array_equal(ref, got)


def test_noalloc_refuses_what_the_scratch_cannot_hold(gpu):
    plan = AG.GemmPlan.create(512, 4096, 14336, "bf16", "bf16")
    assert plan.workspace_bytes() > _capi.NOALLOC_SCRATCH_BYTES
    with pytest.raises(_capi.AsterGemmError) as err:
        plan.run_noalloc(256, 256, 256)     # refused before any pointer is used
    assert err.value.code == -22 and "scratch" in str(err.value)


def test_caller_workspace_matches_the_library_workspace(gpu):
    M, N, K = 96, 1000, 16384
    rng = np.random.default_rng(11)
    a, b = _bf16(rng, (M, K), 1.0), _bf16(rng, (N, K), 0.02)
    plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16")
    need = plan.workspace_bytes()
    assert need > 0
    bufs = [GpuBuffer(a.nbytes), GpuBuffer(b.nbytes), GpuBuffer(M * N * 2), GpuBuffer(need)]
    bufs[0].copy_from_host(a)
    bufs[1].copy_from_host(b)
    out_lib, out_own = np.zeros((M, N), np.uint16), np.zeros((M, N), np.uint16)
    plan.run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2].ptr_value)
    bufs[2].copy_to_host(out_lib)
    plan.run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2].ptr_value, workspace=bufs[3].ptr_value,
             workspace_bytes=need)
    bufs[2].copy_to_host(out_own)
    assert np.array_equal(out_lib, out_own)
    with pytest.raises(_capi.AsterGemmError):
        plan.run(bufs[0].ptr_value, bufs[1].ptr_value, bufs[2].ptr_value,
                 workspace=bufs[3].ptr_value, workspace_bytes=need - 4)
    for bf in bufs:
        bf.free()


def _hip():
    # the HIP runtime the library itself is linked against, found through the library's own handle
    # (another copy of libamdhip64 may be loaded in this process, e.g. the one torch ships, and a
    # stream of one runtime means nothing to the other)
    lib = _capi.load()
    for name, args in (("hipStreamBeginCapture", [ctypes.c_void_p, ctypes.c_int]),
                       ("hipStreamEndCapture", [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]),
                       ("hipGraphInstantiate", [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p,
                                                ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
                       ("hipGraphLaunch", [ctypes.c_void_p, ctypes.c_void_p]),
                       ("hipGraphExecDestroy", [ctypes.c_void_p]),
                       ("hipGraphDestroy", [ctypes.c_void_p])):
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = args, ctypes.c_int
    return lib


def test_noalloc_launches_replay_from_a_graph(gpu):
    # two decode projections in a row, h = x W1^T (no K ranges) and y = h W2^T (rows cut into K
    # ranges: partial sums in the built-in scratch array), captured once in global capture mode
    # (a hipMalloc or a synchronizing call inside the capture would fail it) and replayed on
    # three different x, with eager launches and synchronizations in between; every replay must
    # give the bits of the eager pair on the same x
    M, H, D = 16, 4096, 14336
    rng = np.random.default_rng(21)
    w1, w2 = _bf16(rng, (D, H), 0.02), _bf16(rng, (H, D), 0.02)
    xs = [_bf16(rng, (M, H), 1.0) for _ in range(3)]
    up = AG.GemmPlan.create(M, D, H, "bf16", "bf16")
    down = AG.GemmPlan.create(M, H, D, "bf16", "bf16")
    assert up.workspace_bytes() == 0 and 0 < down.workspace_bytes() <= _capi.NOALLOC_SCRATCH_BYTES
    dx, dw1, dw2 = GpuBuffer(xs[0].nbytes), GpuBuffer(w1.nbytes), GpuBuffer(w2.nbytes)
    dh, dy = GpuBuffer(M * D * 2), GpuBuffer(M * H * 2)
    dw1.copy_from_host(w1)
    dw2.copy_from_host(w2)
    rt, hip = _capi.load(), _hip()

    def eager_pair(x):
        dx.copy_from_host(x)
        up.run(dx.ptr_value, dw1.ptr_value, dh.ptr_value)
        down.run(dh.ptr_value, dw2.ptr_value, dy.ptr_value)
        y = np.zeros((M, H), np.uint16)
        dy.copy_to_host(y)
        return y

    want = [eager_pair(x) for x in xs]
    assert not np.array_equal(want[0], want[1])
    # the eager calls above were also the first calls on this device: set-up is behind us
    up.run_noalloc(dx.ptr_value, dw1.ptr_value, dh.ptr_value)
    down.run_noalloc(dh.ptr_value, dw2.ptr_value, dy.ptr_value)
    _capi.check(rt.aster_rt_device_synchronize())

    stream, graph, gexec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    _capi.check(rt.aster_rt_stream_create(ctypes.byref(stream)))
    print("capture", up.info.name.decode(), down.info.name.decode(), flush=True)
    assert hip.hipStreamBeginCapture(stream, 0) == 0        # hipStreamCaptureModeGlobal
    try:
        up.run_noalloc(dx.ptr_value, dw1.ptr_value, dh.ptr_value, stream=stream.value)
        down.run_noalloc(dh.ptr_value, dw2.ptr_value, dy.ptr_value, stream=stream.value)
    finally:
        rc = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, 0) == 0
    try:
        for i in (2, 0, 1):
            # eager work between the replays: another x through the allocating entry point
            assert np.array_equal(eager_pair(xs[(i + 1) % 3]), want[(i + 1) % 3])
            dx.copy_from_host(xs[i])
            dy.copy_from_host(np.full((M, H), 0x7FC1, np.uint16))
            print("replay on x", i, flush=True)
            assert hip.hipGraphLaunch(gexec, stream) == 0
            _capi.check(rt.aster_rt_stream_synchronize(stream))
            y = np.zeros((M, H), np.uint16)
            dy.copy_to_host(y)
            assert np.array_equal(y, want[i]), f"replay on x{i}"
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
        _capi.check(rt.aster_rt_stream_destroy(stream))
        for bf in (dx, dw1, dw2, dh, dy):
            bf.free()


_CAPTURE_CHILD = r"""
import ctypes, sys
import numpy as np
from aster_amd import _capi, gemm as AG
from aster_amd.execution import GpuBuffer

lib = _capi.load()
for name, args in (("hipStreamBeginCapture", [ctypes.c_void_p, ctypes.c_int]),
                   ("hipStreamEndCapture", [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]),
                   ("hipGraphInstantiate", [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p,
                                            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
                   ("hipGraphLaunch", [ctypes.c_void_p, ctypes.c_void_p])):
    fn = getattr(lib, name)
    fn.argtypes, fn.restype = args, ctypes.c_int
_capi.check(lib.aster_rt_init())
M, N, K = 16, 4096, 14336                      # rows cut into K ranges: partial sums in the scratch
rng = np.random.default_rng(3)
x = (rng.standard_normal((M, K)).astype(np.float32)).view(np.uint32) >> 16
w = (rng.standard_normal((N, K)).astype(np.float32) * 0.02).view(np.uint32) >> 16
x, w = x.astype(np.uint16), w.astype(np.uint16)
dx, dw, dy = GpuBuffer(x.nbytes), GpuBuffer(w.nbytes), GpuBuffer(M * N * 2)
dx.copy_from_host(x)
dw.copy_from_host(w)
plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16")
stream, graph, gexec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
_capi.check(lib.aster_rt_stream_create(ctypes.byref(stream)))

# 1. nothing of this config has run in this process: its first launch inside a capture is refused
assert lib.hipStreamBeginCapture(stream, 0) == 0
try:
    plan.run_noalloc(dx.ptr_value, dw.ptr_value, dy.ptr_value, stream=stream.value)
    refused = None
except _capi.AsterGemmError as exc:
    refused = str(exc)
rc = lib.hipStreamEndCapture(stream, ctypes.byref(graph))
assert refused and "astergemm_prepare" in refused, refused
print("refused:", refused, flush=True)

# 2. after astergemm_prepare the same capture goes through, and the replay gives the eager bits
plan.prepare()
assert lib.hipStreamBeginCapture(stream, 0) == 0
plan.run_noalloc(dx.ptr_value, dw.ptr_value, dy.ptr_value, stream=stream.value)
assert lib.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0 and graph.value
assert lib.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, 0) == 0
got = []
for _ in range(2):
    dy.copy_from_host(np.full((M, N), 0x7FC1, np.uint16))
    assert lib.hipGraphLaunch(gexec, stream) == 0
    _capi.check(lib.aster_rt_stream_synchronize(stream))
    y = np.zeros((M, N), np.uint16)
    dy.copy_to_host(y)
    got.append(y)
plan.run(dx.ptr_value, dw.ptr_value, dy.ptr_value)
_capi.check(lib.aster_rt_device_synchronize())
eager = np.zeros((M, N), np.uint16)
dy.copy_to_host(eager)
assert np.array_equal(got[0], eager) and np.array_equal(got[1], eager)
print("CAPTURE-OK", flush=True)
"""


def test_first_launch_inside_a_capture_is_refused_until_prepared(gpu):
    # in a process of its own, so that no earlier test has launched the kernel: the first launch of
    # a kernel on a device sets a function attribute, which must not happen inside a capture; the
    # library refuses it and astergemm_prepare does that step ahead of time
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("child process: capture before / after astergemm_prepare", flush=True)
    proc = subprocess.run([sys.executable, "-c", _CAPTURE_CHILD], cwd=root, capture_output=True, text=True,
                          timeout=110)
    assert proc.returncode == 0 and "CAPTURE-OK" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-2000:]
