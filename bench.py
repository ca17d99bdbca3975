#!/usr/bin/env python3
"""Headline benchmark: bf16 GEMM M = N = K = 8192 on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one launch of the GEMM hot path (C[M,N] = A[M,K] . B[N,K]^T, A row-major,
B stored N x K, values N(0,1) * 0.02, fp32 accumulate, bf16 output) through the
C-ABI (`astergemm_run`), operands resident in HBM before the timed region.
Prints ONE JSON line.  `value` = 2*M*N*K*steps / wall time of the timed region, in
TFLOP/s.  `roofline.achieved` = flops per launch / average launch duration taken
from a HIP event pair recorded on the launch stream around the same timed region.
`cpu_baseline` = the reference's CPU check (numpy fp32 `A @ B.T`, all host cores)
on a bounded row sample of the same workload.  `others` carries the remaining
shapes of the metric (fp8 8192^3, MXFP4, skinny M = 1/16/64 with the last-level
cache flushed between launches), each timed with an event pair per launch, p50.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "fp8_e4m3": 5000.0, "mxfp4": 10100.0}
# The MI355X datasheet's dense figures; the reference's own harness table has 2500.0 for gfx950
# (contrib/kittens/test/bench/bench_harness.py:31-37), which is PEAK_TFLOPS above.  Fractions are
# reported against both.
PEAK_TFLOPS_DATASHEET = {"bf16": 2516.6, "f16": 2516.6, "fp8_e4m3": 5033.2, "mxfp4": 10066.3}
PEAK_HBM_GBPS = 8000.0

# Bytes moved past L2 per launch of the 8192^3 workload, by kernel, from two
# `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE; KiB per dispatch, each scaled by what
# the same counter reads for a 1 GiB device-to-device copy: x2.0 and x1.0); the figures
# are in profiles/stream_bf16_8192x8192x8192_counters.txt.  A kernel that has not been
# measured reports null.
MEASURED_TRAFFIC_BYTES = {
    "stream_bf16_256x256_w2x4_bf16": 1.746e9,   # 8192^3: 1.61e9 read + 1.34e8 written
    "stream_fp8_256x256_w2x4_bf16": 9.40e8,     # 8192^3: 8.06e8 read + 1.34e8 written
    "stream_fp8_256x256_w2x4_walk_bf16": 9.47e8,  # 8192^3 as a tile walk: 8.12e8 read + 1.35e8 written
    "streamdb_fp8_128x256_w1x4_bf16": 1.203e9,  # 8192^3, weights pre-shuffled: 1.069e9 read + 1.34e8 written
    "stream_mxfp4_256x256_w2x2_bf16": 3.22e8,   # 4096x14336x4096: 2.05e8 read + 1.17e8 written
    # the MXFP4 rows: operands quantised from N(0,1) on the device, as the bench times them
    "stream_mxfp4_256x256_w2x4_tail128_bf16": 3.18e8,  # the same shape: 2.00e8 read + 1.18e8 written
    "streamdb_mxfp4_128x256_w1x4_bf16": 3.14e8,  # the same shape, weights pre-shuffled: 1.96e8 + 1.17e8
    # the same shape, both e8m0 planes in lane order, operands quantised from N(0,1): 1.99e8 + 1.17e8
    "streamdb_mxfp4_128x256_w1x4_sal_bf16": 3.17e8,
}


def _percentile(sorted_vals, pct):
    n = len(sorted_vals)
    return sorted_vals[max(0, min(n - 1, int(round(pct / 100.0 * (n - 1)))))]


def make_operands(torch, M, N, K, dtype_ab, dev, seed=42):
    """Synthetic operands on the device, in storage form, plus launch keywords."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    keep = {}
    if dtype_ab in ("bf16", "f16"):
        # skinny shapes: activations N(0,1); square shapes: both operands N(0,1) * 0.02
        tdt = torch.bfloat16 if dtype_ab == "bf16" else torch.float16
        a = (torch.randn(M, K, device=dev, generator=g) * (0.02 if M >= 256 else 1.0)).to(tdt)
        g.manual_seed(seed + 1)
        b = (torch.randn(N, K, device=dev, generator=g) * 0.02).to(tdt)
        return a, b, keep
    if dtype_ab == "fp8_e4m3":
        xa = torch.randn(M, K, device=dev, generator=g)
        g.manual_seed(seed + 1)
        xb = torch.randn(N, K, device=dev, generator=g)
        sa = (xa.abs().max() / 448.0).reshape(1).float()
        sb = (xb.abs().max() / 448.0).reshape(1).float()
        a = (xa / sa).to(torch.float8_e4m3fn)
        b = (xb / sb).to(torch.float8_e4m3fn)
        keep = {"scale_a": sa, "scale_b": sb}
        return a, b, keep
    if dtype_ab == "mxfp4":
        # N(0,1) sources quantised on the device (astergemm_quantize_mxfp4): e8m0 from the absmax
        # of every 32-wide K block, e2m1 elements, as the baseline's configuration 5 states
        from aster_amd import quantize as Q

        def quantised(rows):
            x = torch.randn(rows, K, device=dev, generator=g)
            packed = torch.empty(rows, K // 2, device=dev, dtype=torch.uint8)
            scales = torch.empty(rows, K // 32, device=dev, dtype=torch.uint8)
            torch.cuda.synchronize()
            Q.quantize_mxfp4_device(x.data_ptr(), rows, K, packed.data_ptr(), scales.data_ptr())
            torch.cuda.synchronize()
            return packed, scales

        a, sa = quantised(M)
        g.manual_seed(seed + 1)
        b, sb = quantised(N)
        keep = {"mx_a": sa, "mx_b": sb}
        return a, b, keep
    raise ValueError(dtype_ab)


OPERANDS = {
    "bf16": "bf16 of N(0,1) * 0.02 (activations of the skinny shapes: N(0,1))",
    "f16": "f16 of N(0,1) * 0.02",
    "fp8_e4m3": "e4m3 of N(0,1) sources with s = absmax/448",
    "mxfp4": "MXFP4 of N(0,1) sources quantised on the device (e8m0 from per-block absmax)",
}


def board_reading_during(plan, a, b, c, seconds=3.5, sample_at=2.5):
    """Socket power and per-XCD shader clocks as the board itself reports them (`amd-smi metric
    --power --clock`, run as a child process) while `plan` runs back to back: the launches go out
    in one call that returns when they are done; a thread takes the sample `sample_at` seconds in.
    None when the tool is missing or prints something else."""
    import re
    import shutil
    import subprocess
    import threading

    tool = shutil.which("amd-smi") or "/opt/rocm/bin/amd-smi"
    if not os.path.exists(tool):
        return None
    sets = [{"dA": a.data_ptr(), "dB": b.data_ptr(), "dC": c.data_ptr()}]
    per_launch_ns = plan.bench_rotate(sets, 20) / 20.0
    launches = max(20, int(seconds * 1e9 / per_launch_ns))
    got = {}

    def sample():
        time.sleep(sample_at)
        try:
            got["text"] = subprocess.run([tool, "metric", "--power", "--clock"], capture_output=True,
                                         text=True, timeout=20).stdout
        except Exception as e:  # noqa: BLE001 - the reading is optional
            got["error"] = repr(e)

    th = threading.Thread(target=sample)
    th.start()
    total_ns = plan.bench_rotate(sets, launches)
    th.join()
    text = got.get("text", "")
    power = re.search(r"SOCKET_POWER:\s*([0-9.]+)\s*W", text)
    clocks = [int(m) for m in re.findall(r"GFX_\d+:\s*\n\s*CLK:\s*(\d+)\s*MHz", text)]
    if not power or not clocks:
        return None
    return {"socket_power_w": float(power.group(1)), "gfx_clk_mhz": clocks, "gfx_max_clk_mhz": 2400,
            "tflops_during_the_reading": round(plan.info.flops * launches / total_ns * 1e-3, 1),
            "launches": launches, "sampled_after_s": sample_at,
            "source": "amd-smi metric --power --clock, as a child process, while the headline kernel "
                      "runs back to back"}


def event_timed_p50(plan, a, b, c, keep, iters, drop, flush_bytes=0):
    kw = {k: v.data_ptr() for k, v in keep.items()}
    times = plan.bench(a.data_ptr(), b.data_ptr(), c.data_ptr(), iters, flush_bytes=flush_bytes, **kw)
    t = sorted(times[drop:])
    return _percentile(t, 50), t[0], sum(t) / len(t)


def preheat(plan, a, b, c, keep, limit_ms):
    """Untimed launches of `plan` until ten in a row agree within 1 %, for at most `limit_ms`;
    returns how many there were.  After the operand set-up in front of a row the first launches of
    a short kernel run up to 15 % slower than the steady state (clocks settling): without this the
    first kernel timed on a shape pays for the one timed after it."""
    kw = {k: v.data_ptr() for k, v in keep.items()}
    launches, t0 = 0, time.perf_counter()
    while limit_ms > 0 and (time.perf_counter() - t0) * 1e3 < limit_ms:
        last = plan.bench(a.data_ptr(), b.data_ptr(), c.data_ptr(), 10, **kw)
        launches += 10
        if launches >= 30 and max(last) <= 1.01 * min(last):
            break
    return launches


def cpu_baseline(M, N, K, budget_s=12.0):
    """numpy fp32 `A @ B.T` (the reference's CPU check) on a row sample sized to
    about `budget_s` seconds; returns the JSON object.  A second leg times the oracle's plain-C
    restatement (OpenMP, fp32 accumulate) on a smaller row sample of the same workload."""
    import numpy as np

    from oracle import cgemm, formats as F, gemm as G

    cores = int(os.environ.get("OMP_NUM_THREADS") or os.cpu_count() or 1)
    rng = np.random.default_rng(43)
    b = F.f32_to_bf16_bits((rng.standard_normal((N, K), dtype=np.float32) * 0.02))
    bf = G.decode_operand(b, G.BF16)
    rng = np.random.default_rng(42)

    def sample(rows):
        a = F.f32_to_bf16_bits(rng.standard_normal((rows, K), dtype=np.float32) * 0.02)
        t0 = time.perf_counter()
        out = G.gemm_epilogue(G.gemm_f32(G.decode_operand(a, G.BF16), bf), G.BF16)
        return time.perf_counter() - t0, out

    probe_rows = 256
    sample(probe_rows)  # warm the BLAS threads
    t_probe, _ = sample(probe_rows)
    rows = int(min(M, max(probe_rows, probe_rows * budget_s / max(t_probe, 1e-6))))
    rows = max(256, rows // 256 * 256)
    t, _ = sample(rows)
    tflops = 2.0 * rows * N * K / t / 1e12
    out = {"value": round(tflops, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
           "sample": f"numpy fp32 A@B.T + bf16 cast on {rows} of {M} rows of A against the full "
                     f"B ({N}x{K}), {t:.2f} s, BLAS threads={cores}"}
    try:
        def csample(rows):
            a = F.f32_to_bf16_bits(rng.standard_normal((rows, K), dtype=np.float32) * 0.02)
            t0 = time.perf_counter()
            cgemm.gemm_raw(a, b, G.BF16, rows, N, K)
            return time.perf_counter() - t0

        csample(32)  # start the OpenMP threads
        t_probe = csample(32)
        crows = int(min(M, max(32, 32 * 6.0 / max(t_probe, 1e-6)))) // 32 * 32
        tc = csample(crows)
        out["c_restatement"] = {"value": round(2.0 * crows * N * K / tc / 1e12, 4), "unit": "TFLOP/s",
                                "cores": cores, "kind": "port",
                                "sample": f"oracle/cgemm.c (OpenMP, fp32 accumulate, bf16 decode) on "
                                          f"{crows} of {M} rows of A against the full B, {tc:.2f} s, "
                                          f"OMP threads={cores}"}
    except Exception as exc:  # the second leg never fails the bench line
        out["c_restatement"] = {"error": repr(exc)[:200]}
    return out


def vendor_call(torch, a, b, keep, dt):
    """The vendor library's GEMM on operands made by `make_operands` (this build's storage forms:
    e4m3 bytes with one fp32 scale per tensor; e2m1 nibbles, low nibble first, with e8m0 bytes
    [rows, K/32])."""
    if dt in ("bf16", "f16"):
        return lambda: torch.matmul(a, b.t())
    if dt == "fp8_e4m3":
        sa, sb = keep["scale_a"].reshape(()), keep["scale_b"].reshape(())
        return lambda: torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
    a4, b4 = a.view(torch.float4_e2m1fn_x2), b.view(torch.float4_e2m1fn_x2)
    sa, sb = keep["mx_a"].view(torch.float8_e8m0fnu), keep["mx_b"].view(torch.float8_e8m0fnu)
    return lambda: torch._scaled_mm(a4, b4.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)


def vendor_library(torch, dev, iters=100, drop=20, preheat_ms=300.0):
    """The vendor's GEMM (torch.matmul / torch._scaled_mm, which call hipBLASLt) on the headline
    shapes with the same timing protocol (one event pair per launch, p50 after dropping the
    first launches).  Reported beside the build's own numbers as the practical ceiling of the
    box; nothing in the product path uses it."""
    rows = []

    def event_timed(fn, count):
        ts = []
        for _ in range(count):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            fn()
            e.record()
            e.synchronize()
            ts.append(s.elapsed_time(e) * 1e3)
        return ts

    def timed(fn):
        # the same untimed pre-heat this build's own rows get (`preheat`)
        launches, t0 = 0, time.perf_counter()
        while preheat_ms > 0 and (time.perf_counter() - t0) * 1e3 < preheat_ms:
            last = event_timed(fn, 10)
            launches += 10
            if launches >= 30 and max(last) <= 1.01 * min(last):
                break
        for _ in range(drop):
            fn()
        torch.cuda.synchronize()
        ts = sorted(event_timed(fn, iters - drop))
        return _percentile(ts, 50)

    for (m, n, k, dt) in ((8192, 8192, 8192, "bf16"), (8192, 8192, 8192, "fp8_e4m3"),
                          (4096, 14336, 4096, "mxfp4"), (16, 14336, 4096, "bf16")):
        try:
            # the bytes this build's own row of the same shape is timed on (same generator, same
            # seeds, same device quantisers): on a power-limited chip operand values move the clock
            a, b, keep = make_operands(torch, m, n, k, dt, dev)
            fn = vendor_call(torch, a, b, keep, dt)
            us = timed(fn)
            row = {"workload": f"{dt} GEMM {m}x{n}x{k} -> bf16", "library": "hipBLASLt via torch",
                   "operands": OPERANDS[dt],
                   "p50_us": round(us, 2), "tflops": round(2.0 * m * n * k / us * 1e-6, 1)}
            if m <= 64:
                row["gbps"] = round((n * k * 2 + m * k * 2 + m * n * 2) / us * 1e-3, 1)
            rows.append(row)
            del a, b, keep, fn
        except Exception as exc:  # a missing library kernel is not this build's failure
            rows.append({"workload": f"{dt} GEMM {m}x{n}x{k} -> bf16", "error": repr(exc)[:200]})
    return rows


SWEEP_SHAPES = [(1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 1024),
                (4096, 14336, 4096), (8000, 8000, 8000), (512, 8192, 8192), (128, 14336, 4096),
                (256, 14336, 4096), (8192, 1024, 8192), (3000, 5000, 7008), (16384, 16384, 4096),
                # down-projections: decode (K ranges in the resident kernels) and short prefill (split K)
                (16, 4096, 14336), (64, 4096, 14336), (128, 4096, 14336), (512, 4096, 14336),
                (16, 8192, 28672)]


def shape_sweep(torch, dev):
    """`--sweep`: this build next to the vendor library over square, skinny, fat and ragged
    shapes, bf16 and fp8, p50 of event-timed launches.  Prints one line per shape."""
    from aster_amd import gemm as AG

    def vendor(a, b, keep, dt):
        fn = vendor_call(torch, a, b, keep, dt)
        for _ in range(15):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(45):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            fn()
            e.record()
            e.synchronize()
            ts.append(s.elapsed_time(e) * 1e3)
        ts.sort()
        return _percentile(ts, 50)

    rows = []
    for dt in ("bf16", "fp8_e4m3", "mxfp4"):
        for (m, n, k) in SWEEP_SHAPES:
            if dt == "mxfp4" and k % 256:
                continue                    # the MXFP4 kernels take whole 128-byte K steps
            a, b, keep = make_operands(torch, m, n, k, dt, dev)
            c = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
            p = AG.GemmPlan.create(m, n, k, dt, "bf16")
            ours, _, _ = event_timed_p50(p, a, b, c, keep, 60, 15)
            ours /= 1e3
            del c
            try:
                ven = vendor(a, b, keep, dt)
            except Exception as exc:  # shapes the vendor entry point refuses
                ven = None
                note = repr(exc)[:60]
            del a, b, keep
            fl = 2.0 * m * n * k
            row = {"dtype": dt, "M": m, "N": n, "K": k, "kernel": p.info.name.decode(),
                   "us": round(ours, 1), "tflops": round(fl / ours * 1e-6, 1),
                   "vendor_us": None if ven is None else round(ven, 1),
                   "vendor_tflops": None if ven is None else round(fl / ven * 1e-6, 1),
                   "vendor_over_ours": None if ven is None else round(ven / ours, 2)}
            rows.append(row)
            print(f"{dt:9s} {m:6d}x{n:6d}x{k:6d}  {row['us']:9.1f} us {row['tflops']:7.1f} TF   vendor "
                  + (f"{row['vendor_us']:9.1f} us {row['vendor_tflops']:7.1f} TF  x{row['vendor_over_ours']:.2f}"
                     if ven is not None else f"refused ({note})")
                  + f"   {row['kernel']}", flush=True)
    return rows


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--preheat-ms", type=float, default=1500.0,
                    help="upper bound of the untimed pre-heat of the headline kernel before the "
                         "warm-up launches (0 = none)")
    ap.add_argument("--no-others", action="store_true", help="skip the secondary shapes")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-board", action="store_true",
                    help="skip the power / clock reading (3.5 s of back-to-back launches)")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip timing the vendor library (hipBLASLt through torch) on the same shapes")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the bench line: time a list of shapes here and in the vendor "
                         "library, one text line per shape and one JSON line at the end")
    ap.add_argument("--results-jsonl", default=None,
                    help="also append one BENCH_RESULT_JSON line per MFMA-bound workload to this "
                         "file (input of `python -m aster_amd.perf_registry`)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(the path would shard over GPUs by splitting B's rows, one slice of C per GPU, no communication)", file=sys.stderr)
        return 2

    import torch

    from aster_amd import _capi, gemm as AG

    _capi.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    lib = _capi.load()
    if args.sweep:
        print(json.dumps({"sweep": shape_sweep(torch, dev)}), flush=True)
        return 0

    M = N = K = 8192
    a, b, keep = make_operands(torch, M, N, K, "bf16", dev)
    c = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    plan = AG.GemmPlan.create(M, N, K, "bf16", "bf16")
    flops = float(plan.info.flops)

    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _capi.check(lib.aster_rt_event_create(ctypes.byref(e0)))
    _capi.check(lib.aster_rt_event_create(ctypes.byref(e1)))

    # the same timed region once BEFORE anything has warmed the chip (no MFMA-rate loop, no pre-heat,
    # no warm-up launches): what a caller sees on the first launches after idling
    torch.cuda.synchronize()
    t_cold = time.perf_counter()
    for _ in range(args.steps):
        plan.run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    cold_wall = time.perf_counter() - t_cold

    # what the matrix pipe alone sustains on these operand values under the power limit
    # (independent MFMAs over registers filled from B, no memory traffic), measured first so that
    # its 300 ms also bring the clocks to their loaded state
    ceil_tf = AG.mfma_rate(b.data_ptr(), b.numel() * b.element_size(), "bf16", target_ms=300)

    # Untimed pre-heat of the same kernel: after idling, the first launches run up to a third
    # slower than the steady state (clock and power management settling), which a short timed
    # region right after a short warm-up would otherwise sit in.  Launches are event-timed one by
    # one until ten in a row agree within 1 %, for at most `--preheat-ms`.
    preheat_launches, t_pre = 0, time.perf_counter()
    if args.preheat_ms > 0:
        recent = []
        while (time.perf_counter() - t_pre) * 1e3 < args.preheat_ms:
            recent += plan.bench(a.data_ptr(), b.data_ptr(), c.data_ptr(), 10)
            preheat_launches += 10
            last = recent[-10:]
            if preheat_launches >= 30 and max(last) <= 1.01 * min(last):
                break
    preheat_ms = (time.perf_counter() - t_pre) * 1e3

    for _ in range(args.warmup):
        plan.run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    _capi.check(lib.aster_rt_event_record(e0, None))
    for _ in range(args.steps):
        plan.run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    _capi.check(lib.aster_rt_event_record(e1, None))
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = ctypes.c_float()
    _capi.check(lib.aster_rt_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    launch_ms = ms.value / args.steps
    value = flops * args.steps / wall / 1e12
    achieved = flops / (launch_ms * 1e-3) / 1e12
    # the reference's protocol beside it: one event pair per launch, 100 launches, first 20
    # dropped, p50 (bench_harness.py:93-94, 181-198)
    p50_ns, p0_ns, _ = event_timed_p50(plan, a, b, c, keep, 100, 20)

    traffic = MEASURED_TRAFFIC_BYTES.get(plan.info.name.decode())

    out = {
        "metric": "bf16 GEMM 8192^3 throughput (TFLOP/s; % of MI355X dense MFMA peak in roofline.frac)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "preheat_ms": round(preheat_ms, 1), "preheat_launches": preheat_launches,
        "value_first_launches_after_idle": round(flops * args.steps / cold_wall / 1e12, 2),
        "p50_us": round(p50_ns / 1e3, 2), "p50_tflops": round(flops / p50_ns * 1e-3, 1),
        "config": {"workload": "bf16 GEMM M=N=K=8192, A row-major, B stored NxK (column-major KxN), "
                               "N(0,1)*0.02, fp32 accumulate, bf16 output",
                   "kernel": plan.info.name.decode(), "grid": plan.info.grid_x,
                   "block": plan.info.block_x, "lds_bytes": plan.info.lds_bytes},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["bf16"],
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_TFLOPS["bf16"], 4),
                     "traffic": traffic,
                     "peak_datasheet": PEAK_TFLOPS_DATASHEET["bf16"],
                     "frac_of_datasheet_peak": round(achieved / PEAK_TFLOPS_DATASHEET["bf16"], 4)},
    }
    out["roofline"]["mfma_rate_measured_on_this_data"] = round(ceil_tf, 1)
    out["roofline"]["frac_of_measured_mfma_rate"] = round(achieved / ceil_tf, 4)
    # what the board says while this kernel runs (behind the timed region, so it costs it nothing)
    out["board"] = None if args.no_board else board_reading_during(plan, a, b, c)

    if not args.no_others:
        others = []
        # the headline product on the reference's other operand paths: B pre-shuffled and loaded
        # straight into MFMA operands (direct_b), A and B both (direct_ab, no LDS); shuffled once,
        # on the device
        from aster_amd import quantize as Q
        others_preheat_ms = min(args.preheat_ms, 300.0)
        for path in ("direct_b_k8", "direct_ab"):
            a_s = a
            if path == "direct_ab":
                a_s = torch.empty_like(a)
            b_s = torch.empty_like(b)
            c_s = torch.empty_like(c)
            torch.cuda.synchronize()
            if path == "direct_ab":
                Q.preshuffle_device(a.data_ptr(), a_s.data_ptr(), M, K, "bf16", path)
            Q.preshuffle_device(b.data_ptr(), b_s.data_ptr(), N, K, "bf16", path)
            torch.cuda.synchronize()
            pp = AG.GemmPlan.create(M, N, K, "bf16", "bf16", operand_path=path)
            pre = preheat(pp, a_s, b_s, c_s, {}, others_preheat_ms)
            p50, _, _ = event_timed_p50(pp, a_s, b_s, c_s, {}, 100, 20)
            tf = pp.info.flops / p50 * 1e-3
            diff = (c_s.float() - c.float()).norm() / c.float().norm()
            others.append({"workload": f"bf16 GEMM {M}x{N}x{K} -> bf16, operand_path {path.replace('_k8', '')}",
                           "operands": OPERANDS["bf16"], "kernel": pp.info.name.decode(),
                           "preheat_launches": pre, "p50_us": round(p50 / 1e3, 2),
                           "tflops": round(tf, 1), "bound": "mfma",
                           "frac": round(tf / PEAK_TFLOPS["bf16"], 4),
                           "rel_l2_to_the_headline_output": float(diff)})
            del a_s, b_s, c_s
        for (m, n, k, dt) in ((8192, 8192, 8192, "fp8_e4m3"), (4096, 14336, 4096, "mxfp4")):
            del a, b, c
            a, b, keep = make_operands(torch, m, n, k, dt, dev)
            c = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
            p = AG.GemmPlan.create(m, n, k, dt, "bf16")
            pre = preheat(p, a, b, c, keep, others_preheat_ms)
            p50, best, _ = event_timed_p50(p, a, b, c, keep, 100, 20)
            tf = p.info.flops / p50 * 1e-3
            ceil_tf = AG.mfma_rate(b.data_ptr(), b.numel() * b.element_size(), dt, target_ms=200)
            others.append({"workload": f"{dt} GEMM {m}x{n}x{k} -> bf16", "operands": OPERANDS[dt],
                           "kernel": p.info.name.decode(), "preheat_launches": pre,
                           "p50_us": round(p50 / 1e3, 2), "tflops": round(tf, 1), "bound": "mfma",
                           "frac": round(tf / PEAK_TFLOPS[dt], 4),
                           "frac_of_datasheet_peak": round(tf / PEAK_TFLOPS_DATASHEET[dt], 4),
                           "algorithmic_bytes": int(p.info.bytes),
                           "traffic": MEASURED_TRAFFIC_BYTES.get(p.info.name.decode()),
                           "mfma_rate_measured_on_this_data": round(ceil_tf, 1),
                           "frac_of_measured_mfma_rate": round(tf / ceil_tf, 4)})
            # the same product with the weights pre-shuffled (operand_path direct_b_k8: payload
            # in step order, the MXFP4 e8m0 plane in lane order), the way the reference's best
            # kernel takes its B; shuffled once, on the device (astergemm_preshuffle)
            bs = torch.empty_like(b)
            sbs = torch.empty_like(keep["mx_b"]) if dt == "mxfp4" else None
            torch.cuda.synchronize()
            Q.preshuffle_device(b.data_ptr(), bs.data_ptr(), n, k, dt, "direct_b_k8",
                                d_mx_src=keep["mx_b"].data_ptr() if sbs is not None else None,
                                d_mx_dst=sbs.data_ptr() if sbs is not None else None)
            torch.cuda.synchronize()
            pd = AG.GemmPlan.create(m, n, k, dt, "bf16", operand_path="direct_b_k8")
            c2 = torch.empty_like(c)
            keep_d = dict(keep, mx_b=sbs) if sbs is not None else keep
            pre_d = preheat(pd, a, bs, c2, keep_d, others_preheat_ms)
            p50d, _, _ = event_timed_p50(pd, a, bs, c2, keep_d, 100, 20)
            tfd = pd.info.flops / p50d * 1e-3
            others[-1].update({"kernel_weights_pre_shuffled": pd.info.name.decode(),
                               "preheat_launches_weights_pre_shuffled": pre_d,
                               "p50_us_weights_pre_shuffled": round(p50d / 1e3, 2),
                               "tflops_weights_pre_shuffled": round(tfd, 1),
                               "frac_weights_pre_shuffled": round(tfd / PEAK_TFLOPS[dt], 4),
                               "traffic_weights_pre_shuffled": MEASURED_TRAFFIC_BYTES.get(pd.info.name.decode()),
                               "same_bits_as_row_major_weights": bool(torch.equal(c, c2))})
            if dt == "mxfp4":
                # and with the activations' e8m0 plane in lane order as well (mx_a_layout lanes128:
                # what the device quantiser writes with scales_layout="lanes128"; here made from the
                # row-major plane by the device pre-shuffle), no scale traffic through LDS
                from aster_amd.kittens_helpers import mx_lanes128_bytes
                sal = torch.empty(mx_lanes128_bytes(m, k), device=dev, dtype=torch.uint8)
                torch.cuda.synchronize()
                Q.preshuffle_scales_a_device(keep["mx_a"].data_ptr(), sal.data_ptr(), m, k)
                torch.cuda.synchronize()
                pl = AG.GemmPlan.create(m, n, k, dt, "bf16", operand_path="direct_b_k8", mx_a_layout="lanes128")
                c3 = torch.empty_like(c)
                keep_l = dict(mx_a=sal, mx_b=sbs)
                pre_l = preheat(pl, a, bs, c3, keep_l, others_preheat_ms)
                p50l, _, _ = event_timed_p50(pl, a, bs, c3, keep_l, 100, 20)
                tfl = pl.info.flops / p50l * 1e-3
                others[-1].update({"kernel_scales_in_lane_order": pl.info.name.decode(),
                                   "preheat_launches_scales_in_lane_order": pre_l,
                                   "p50_us_scales_in_lane_order": round(p50l / 1e3, 2),
                                   "tflops_scales_in_lane_order": round(tfl, 1),
                                   "frac_scales_in_lane_order": round(tfl / PEAK_TFLOPS[dt], 4),
                                   "traffic_scales_in_lane_order": MEASURED_TRAFFIC_BYTES.get(pl.info.name.decode()),
                                   "scales_in_lane_order_same_bits": bool(torch.equal(c, c3))})
                del sal, c3
            del bs, sbs, c2
        # the two gfx950 shapes the reference publishes its own kernels' numbers for (f16
        # operands, fp32 output; contrib/kittens/test/bench/best_known.json, quoted, not re-run)
        for (m, n, k, quoted) in ((4096, 4096, 4096, 1007.0), (2048, 4096, 4096, 846.3)):
            del a, b, c
            a, b, keep = make_operands(torch, m, n, k, "f16", dev)
            c = torch.empty(m, n, device=dev, dtype=torch.float32)
            p = AG.GemmPlan.create(m, n, k, "f16", "f32")
            pre = preheat(p, a, b, c, keep, others_preheat_ms)
            p50, _, _ = event_timed_p50(p, a, b, c, keep, 100, 20)
            tf = p.info.flops / p50 * 1e-3
            others.append({"workload": f"f16 GEMM {m}x{n}x{k} -> f32 (the reference's published shape)",
                           "kernel": p.info.name.decode(), "preheat_launches": pre,
                           "p50_us": round(p50 / 1e3, 2),
                           "tflops": round(tf, 1), "bound": "mfma",
                           "frac": round(tf / PEAK_TFLOPS["bf16"], 4),
                           "reference_quoted_tflops": quoted})
        for m in (1, 16, 64):
            del a, b, c
            a, b, keep = make_operands(torch, m, 14336, 4096, "bf16", dev)
            c = torch.empty(m, 14336, device=dev, dtype=torch.bfloat16)
            p = AG.GemmPlan.create(m, 14336, 4096, "bf16", "bf16")
            p50, best, _ = event_timed_p50(p, a, b, c, keep, 100, 20, flush_bytes=512 << 20)
            hot, _, _ = event_timed_p50(p, a, b, c, keep, 100, 20)
            gbs = p.info.bytes / p50
            # steady state: 8 distinct weight matrices (8 x 112 MiB, 3.5x the last-level
            # cache) used in turn by back-to-back launches inside one event pair
            wts = [b] + [torch.empty_like(b).copy_(b) for _ in range(7)]
            sets = [{"dA": a.data_ptr(), "dB": w.data_ptr(), "dC": c.data_ptr()} for w in wts]
            p.bench_rotate(sets, 40)
            rot_ns = p.bench_rotate(sets, 200) / 200.0
            # the same 200 launches as 5 replays of a captured HIP graph of 40 kernel nodes
            graph_ns = p.bench_graph(sets, 40, 5) / 200.0
            del wts, sets
            others.append({"workload": f"bf16 skinny GEMM M={m} N=14336 K=4096 -> bf16, LLC flushed "
                                       "(512 MiB rewritten) before every launch",
                           "kernel": p.info.name.decode(), "p50_us": round(p50 / 1e3, 2),
                           "gbps": round(gbs, 1), "bound": "hbm",
                           "frac": round(gbs / PEAK_HBM_GBPS, 4),
                           "p50_us_cache_warm": round(hot / 1e3, 2),
                           "us_back_to_back_8_weight_sets": round(rot_ns / 1e3, 2),
                           "gbps_back_to_back": round(p.info.bytes / rot_ns, 1),
                           "frac_back_to_back": round(p.info.bytes / rot_ns / PEAK_HBM_GBPS, 4),
                           "us_graph_replay_8_weight_sets": round(graph_ns / 1e3, 2),
                           "frac_graph_replay": round(p.info.bytes / graph_ns / PEAK_HBM_GBPS, 4)})
        # the decode shape with quantised weights and activations (same kernel frame)
        for dt in ("fp8_e4m3", "mxfp4"):
            del a, b, c
            a, b, keep = make_operands(torch, 16, 14336, 4096, dt, dev)
            c = torch.empty(16, 14336, device=dev, dtype=torch.bfloat16)
            p = AG.GemmPlan.create(16, 14336, 4096, dt, "bf16")
            p50, _, _ = event_timed_p50(p, a, b, c, keep, 100, 20, flush_bytes=512 << 20)
            nsets = 12 if dt == "fp8_e4m3" else 24      # > 2.5x the last-level cache in all
            wts = [b] + [torch.empty_like(b).copy_(b) for _ in range(nsets - 1)]
            kw = {k: v.data_ptr() for k, v in keep.items()}
            sets = [dict(dA=a.data_ptr(), dB=w.data_ptr(), dC=c.data_ptr(), **kw) for w in wts]
            p.bench_rotate(sets, 48)
            rot_ns = p.bench_rotate(sets, 240) / 240.0
            # the same weights pre-shuffled on the device into the MFMA's operand order
            # (operand_path direct_b)
            from aster_amd import quantize as Q
            pd = AG.GemmPlan.create(16, 14336, 4096, dt, "bf16", operand_path="direct_b")
            bs = torch.empty_like(b)
            sbs = torch.empty_like(keep["mx_b"]) if dt == "mxfp4" else None
            torch.cuda.synchronize()
            Q.preshuffle_device(b.data_ptr(), bs.data_ptr(), 14336, 4096, dt, "direct_b",
                                d_mx_src=keep["mx_b"].data_ptr() if sbs is not None else None,
                                d_mx_dst=sbs.data_ptr() if sbs is not None else None)
            torch.cuda.synchronize()
            del wts, sets
            wts = [bs] + [torch.empty_like(bs).copy_(bs) for _ in range(nsets - 1)]
            kwd = dict(kw, mx_b=sbs.data_ptr()) if sbs is not None else kw
            c2 = torch.empty_like(c)
            sets = [dict(dA=a.data_ptr(), dB=w.data_ptr(), dC=c2.data_ptr(), **kwd) for w in wts]
            pd.bench_rotate(sets, 48)
            rot_d_ns = pd.bench_rotate(sets, 240) / 240.0
            p.run(a.data_ptr(), b.data_ptr(), c.data_ptr(), **kw)
            torch.cuda.synchronize()
            same_d = bool(torch.equal(c, c2))
            del wts, sets, bs, sbs, c2
            others.append({"workload": f"{dt} skinny GEMM M=16 N=14336 K=4096 -> bf16, LLC flushed "
                                       "before every launch",
                           "kernel": p.info.name.decode(), "p50_us": round(p50 / 1e3, 2),
                           "gbps": round(p.info.bytes / p50, 1), "bound": "hbm",
                           "frac": round(p.info.bytes / p50 / PEAK_HBM_GBPS, 4),
                           f"us_back_to_back_{nsets}_weight_sets": round(rot_ns / 1e3, 2),
                           "gbps_back_to_back": round(p.info.bytes / rot_ns, 1),
                           "frac_back_to_back": round(p.info.bytes / rot_ns / PEAK_HBM_GBPS, 4),
                           "kernel_weights_pre_shuffled": pd.info.name.decode(),
                           "us_back_to_back_weights_pre_shuffled": round(rot_d_ns / 1e3, 2),
                           "weights_pre_shuffled_same_bits": same_d})
        # the same M = 16 shape with the weights pre-shuffled into MFMA operand order
        # (the reference's operand_path = direct_b), shuffled on the device
        del a, b, c
        a, b, keep = make_operands(torch, 16, 14336, 4096, "bf16", dev)
        c = torch.empty(16, 14336, device=dev, dtype=torch.bfloat16)
        p = AG.GemmPlan.create(16, 14336, 4096, "bf16", "bf16", operand_path="direct_b")
        from aster_amd import quantize as Q
        bs = torch.empty_like(b)
        torch.cuda.synchronize()
        Q.preshuffle_device(b.data_ptr(), bs.data_ptr(), 14336, 4096, "bf16", "direct_b")
        torch.cuda.synchronize()
        b = bs
        p50, _, _ = event_timed_p50(p, a, b, c, keep, 100, 20, flush_bytes=512 << 20)
        wts = [b] + [torch.empty_like(b).copy_(b) for _ in range(7)]
        sets = [{"dA": a.data_ptr(), "dB": w.data_ptr(), "dC": c.data_ptr()} for w in wts]
        p.bench_rotate(sets, 40)
        rot_ns = p.bench_rotate(sets, 200) / 200.0
        del wts, sets
        others.append({"workload": "bf16 skinny GEMM M=16 N=14336 K=4096 -> bf16, weights pre-shuffled "
                                   "(operand_path direct_b), LLC flushed before every launch",
                       "kernel": p.info.name.decode(), "p50_us": round(p50 / 1e3, 2),
                       "gbps": round(p.info.bytes / p50, 1), "bound": "hbm",
                       "frac": round(p.info.bytes / p50 / PEAK_HBM_GBPS, 4),
                       "us_back_to_back_8_weight_sets": round(rot_ns / 1e3, 2),
                       "gbps_back_to_back": round(p.info.bytes / rot_ns, 1),
                       "frac_back_to_back": round(p.info.bytes / rot_ns / PEAK_HBM_GBPS, 4)})
        # the down-projection of the same layer (rows of 28 KiB: the decode kernels run it in
        # K ranges), with the vendor library's time for the same rotation of weight sets
        for m in (16, 64):
            del a, b, c
            a, b, keep = make_operands(torch, m, 4096, 14336, "bf16", dev)
            c = torch.empty(m, 4096, device=dev, dtype=torch.bfloat16)
            p = AG.GemmPlan.create(m, 4096, 14336, "bf16", "bf16")
            wts = [b] + [torch.empty_like(b).copy_(b) for _ in range(7)]
            sets = [{"dA": a.data_ptr(), "dB": w.data_ptr(), "dC": c.data_ptr()} for w in wts]
            p.bench_rotate(sets, 40)
            rot_ns = p.bench_rotate(sets, 200) / 200.0
            entry = {"workload": f"bf16 skinny GEMM M={m} N=4096 K=14336 -> bf16 (down-projection), "
                                 "8 weight sets used in turn",
                     "kernel": p.info.name.decode(), "us_back_to_back_8_weight_sets": round(rot_ns / 1e3, 2),
                     "gbps_back_to_back": round(p.info.bytes / rot_ns, 1), "bound": "hbm",
                     "frac_back_to_back": round(p.info.bytes / rot_ns / PEAK_HBM_GBPS, 4)}
            if not args.no_vendor:
                for i in range(16):
                    torch.matmul(a, wts[i % 8].t())
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for i in range(200):
                    torch.matmul(a, wts[i % 8].t())
                e1.record()
                e1.synchronize()
                entry["vendor_library_us_same_rotation"] = round(e0.elapsed_time(e1) * 1e3 / 200, 2)
            del wts, sets
            others.append(entry)
        # a short prefill through the same down-projection: few output tiles, long rows (split K)
        for dt in ("bf16", "fp8_e4m3"):
            del a, b, c
            a, b, keep = make_operands(torch, 128, 4096, 14336, dt, dev)
            c = torch.empty(128, 4096, device=dev, dtype=torch.bfloat16)
            p = AG.GemmPlan.create(128, 4096, 14336, dt, "bf16")
            p50, _, _ = event_timed_p50(p, a, b, c, keep, 100, 20)
            tf = p.info.flops / p50 * 1e-3
            others.append({"workload": f"{dt} GEMM 128x4096x14336 -> bf16 (32 output tiles of 128x128)",
                           "kernel": p.info.name.decode(), "grid": p.info.grid_x,
                           "p50_us": round(p50 / 1e3, 2), "tflops": round(tf, 1),
                           "gbps": round(p.info.bytes / p50, 1), "bound": "hbm",
                           "frac": round(p.info.bytes / p50 / PEAK_HBM_GBPS, 4)})
        out["others"] = others

    if not args.no_vendor:
        del a, b, c
        out["vendor_library"] = vendor_library(torch, dev, preheat_ms=min(args.preheat_ms, 300.0))

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(M, N, K)
    else:
        out["cpu_baseline"] = None

    if args.results_jsonl:
        from aster_amd.perf_registry import RESULT_SENTINEL
        recs = [("astergemm_bf16", 8192, 8192, 8192, plan.info.name.decode(), achieved)]
        for o in out.get("others", []):
            if o.get("bound") != "mfma":
                continue
            dt = o["workload"].split()[0]
            m, n, k = (int(x) for x in o["workload"].split()[2].split("x"))
            recs.append((f"astergemm_{dt}", m, n, k, o["kernel"], o["tflops"]))
        with open(args.results_jsonl, "a") as f:
            for bench, m, n, k, label, tf in recs:
                f.write(RESULT_SENTINEL + json.dumps({"mcpu": "gfx950", "bench": bench, "M": m, "N": n,
                                                       "K": k, "label": label, "tflops_median": tf,
                                                       "sample_n": 1}) + "\n")
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
