"""Measurement contract of the GEMM benches: input init, stats, single-config run,
result lines.

Mirrors the parts of the reference's bench harness that define what is measured
(contrib/kittens/test/bench/bench_harness.py: peak table :31-41, `InitMode` /
`init_array` :44-90, iteration counts :93-94, `PerfStats` :100-172,
`_percentile_ns` / `_compute_stats` :174-198, `make_inputs` :1655-1662,
`run_single` :1738-1850) and the `BENCH_RESULT_JSON:` line
(tools/perf_bench_results_io.py:15, 113-144).  The compile pool, GPU workers and
tiered config search of that file drive the reference's compiler and have no
counterpart here; `bench_perf_sweep` is the sweep in this build's terms: mappings -> select ->
time -> result lines -> registry dashboard, in one process and one command
(`python -m aster_amd.bench_harness --m ... --n ... --k ...`).
"""

from __future__ import annotations

import enum
import json
import statistics
import sys
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

from .gemm_config import A as OP_A, B as OP_B

# Dense peak TFLOP/s per target and operand type.  The f16 column is the
# reference's table (:31-37); the others are MI355X's published dense peaks.
_PEAK_TFLOPS_F16_BY_MCPU = {"gfx940": 980.6, "gfx942": 1307.0, "gfx950": 2500.0, "gfx1201": 100.0}
PEAK_TFLOPS_GFX950 = {"f16": 2500.0, "bf16": 2500.0, "fp8_e4m3": 5000.0, "mxfp4": 10100.0}
PEAK_HBM_GBPS_GFX950 = 8000.0


def peak_tflops_f16(mcpu: str) -> float:
    return _PEAK_TFLOPS_F16_BY_MCPU[mcpu]


def peak_tflops(mcpu: str, dtype_ab: str = "f16") -> float:
    if mcpu == "gfx950":
        return PEAK_TFLOPS_GFX950[dtype_ab]
    return peak_tflops_f16(mcpu)


class InitMode(str, enum.Enum):
    """Input init modes (hipblas names): HPL uniform[-0.5, 0.5]; TRIG_FLOAT
    A=sin(i), B=cos(i); RAND_INT integers in {-2..2}; ZERO; SPECIAL fp16 extremes
    (A = 65280, B = 6.07967e-5); NORM_DIST N(0, 1)."""

    HPL = "hpl"
    TRIG_FLOAT = "trig_float"
    RAND_INT = "rand_int"
    ZERO = "zero"
    SPECIAL = "special"
    NORM_DIST = "norm_dist"

    def __str__(self) -> str:
        return self.value


INIT_DEFAULT = InitMode.HPL
_SPECIAL = {"A": np.float16(65280.0), "B": np.float16(6.07967376708984375e-5)}

NUM_ITERATIONS = 100
WARMUP_ITERATIONS = 20


def init_array(shape, mode, role: str, dtype=np.float16, seed: int = 42) -> np.ndarray:
    """Deterministic input of the given mode; B uses stream `seed + 1`."""
    mode = InitMode(mode)
    flat = int(np.prod(shape))
    if mode is InitMode.ZERO:
        return np.zeros(shape, dtype=dtype)
    if mode is InitMode.TRIG_FLOAT:
        idx = np.arange(flat, dtype=np.float64)
        return (np.sin(idx) if role == "A" else np.cos(idx)).astype(dtype).reshape(shape)
    if mode is InitMode.SPECIAL:
        return np.full(shape, _SPECIAL["A" if role == "A" else "B"], dtype=dtype)
    rng = np.random.default_rng(seed + (1 if role == "B" else 0))
    if mode is InitMode.HPL:
        vals = rng.uniform(-0.5, 0.5, size=flat)
    elif mode is InitMode.RAND_INT:
        vals = rng.integers(-2, 3, size=flat)
    else:
        vals = rng.standard_normal(size=flat)
    return vals.astype(dtype).reshape(shape)


@dataclass(frozen=True)
class PerfStats:
    p0_ns: float
    p10_ns: float
    p25_ns: float
    p50_ns: float
    p90_ns: float
    mean_ns: float
    stddev_ns: float
    stddev_tf: float
    total_flops: int
    peak_tflops: float

    def _tf(self, ns: float) -> float:
        return self.total_flops / ns * 1e-3

    p0_ms = property(lambda s: s.p0_ns / 1e6)
    p10_ms = property(lambda s: s.p10_ns / 1e6)
    p25_ms = property(lambda s: s.p25_ns / 1e6)
    p50_ms = property(lambda s: s.p50_ns / 1e6)
    p90_ms = property(lambda s: s.p90_ns / 1e6)
    mean_ms = property(lambda s: s.mean_ns / 1e6)
    p0_tf = property(lambda s: s._tf(s.p0_ns))
    p10_tf = property(lambda s: s._tf(s.p10_ns))
    p25_tf = property(lambda s: s._tf(s.p25_ns))
    p50_tf = property(lambda s: s._tf(s.p50_ns))
    p90_tf = property(lambda s: s._tf(s.p90_ns))
    mean_tf = property(lambda s: s._tf(s.mean_ns))
    p0_pct = property(lambda s: s.p0_tf / s.peak_tflops * 100)
    p50_pct = property(lambda s: s.p50_tf / s.peak_tflops * 100)
    mean_pct = property(lambda s: s.mean_tf / s.peak_tflops * 100)


def _percentile_ns(sorted_times: Sequence[float], pct: float) -> float:
    """Nearest-rank percentile of an ascending list."""
    n = len(sorted_times)
    return float(sorted_times[max(0, min(n - 1, int(round(pct / 100.0 * (n - 1)))))])


def _compute_stats(post_warmup: Sequence[float], total_flops: int,
                   peak_tflops: float) -> Optional[PerfStats]:
    """Post-warm-up launch times (ns) -> percentiles, mean, stddev; None when a
    time is not positive."""
    if not post_warmup or min(post_warmup) <= 0:
        return None
    times = sorted(float(t) for t in post_warmup)
    tfs = [int(total_flops) / t * 1e-3 for t in times]
    many = len(times) > 1
    return PerfStats(
        p0_ns=times[0], p10_ns=_percentile_ns(times, 10), p25_ns=_percentile_ns(times, 25),
        p50_ns=_percentile_ns(times, 50), p90_ns=_percentile_ns(times, 90),
        mean_ns=float(statistics.fmean(times)),
        stddev_ns=float(statistics.stdev(times)) if many else 0.0,
        stddev_tf=float(statistics.stdev(tfs)) if many else 0.0,
        total_flops=int(total_flops), peak_tflops=peak_tflops)


RESULT_SENTINEL = "BENCH_RESULT_JSON:"


def emit_one_result(stream, bench: str, cfg, stats: PerfStats, *, label: str = None) -> None:
    """One `BENCH_RESULT_JSON:{...}` line; `stream=None` discards.  `label` replaces the
    config's own label (run_single passes the name of the kernel that actually ran when the
    mapping was not honoured, so that mappings which ran the same pre-built kernel do not
    become separate registry entries)."""
    if stream is None:
        return
    m, n, k = cfg.spec.gemm_size
    rec = {"mcpu": cfg.mapping.mcpu, "bench": bench, "M": m, "N": n, "K": k,
           "label": label or cfg.label,
           "tflops_median": stats.p50_tf, "tflops_p10": stats.p10_tf, "tflops_p90": stats.p90_tf,
           "tflops_mean": stats.mean_tf, "tflops_p0": stats.p0_tf, "tflops_p25": stats.p25_tf,
           "tflops_stddev": stats.stddev_tf, "pct_peak_p50": stats.p50_pct, "sample_n": 1}
    print(RESULT_SENTINEL + json.dumps(rec), file=stream)
    stream.flush()


def parse_result_lines(lines):
    """Records of every `BENCH_RESULT_JSON:` line in `lines`; other text is skipped."""
    out = []
    for raw in lines:
        i = raw.find(RESULT_SENTINEL)
        if i < 0:
            continue
        try:
            out.append(json.loads(raw[i + len(RESULT_SENTINEL):]))
        except json.JSONDecodeError:
            continue
    return out


def _storage(values: np.ndarray, dtype_ab: str) -> np.ndarray:
    """fp16-valued init data in the operand's storage type."""
    if dtype_ab == "f16":
        return values.astype(np.float16)
    if dtype_ab == "bf16":
        u = values.astype(np.float32).view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    raise ValueError(f"make_inputs covers f16 and bf16, not {dtype_ab}")


def make_inputs(cfg, init_mode=INIT_DEFAULT):
    """A [M, K] and B [N, K] for `cfg`, seeds 42 / 43."""
    a = init_array(cfg.spec.operand_shape(OP_A), init_mode, "A")
    b = init_array(cfg.spec.operand_shape(OP_B), init_mode, "B")
    dt = cfg.spec.dtype_ab
    return _storage(a, dt), _storage(b, dt)


def _as_f32(arr: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return (arr.astype(np.uint32) << 16).view(np.float32)
    return arr.astype(np.float32)


def run_single(cfg, compile_fn, args, execute_fn, *, bench: str = "unknown", out=sys.stdout):
    """Compile (select), time `iterations` launches, print the summary table, then
    a one-launch correctness check against `A.f32 @ B.f32.T` with rtol = atol =
    1e-2, as the reference does.  Returns the PerfStats (None without a GPU)."""
    import tempfile

    from .execution import system_has_gpu

    iterations = getattr(args, "iterations", None) or NUM_ITERATIONS
    hsaco = getattr(args, "hsaco", None)
    tmp = None
    if not hsaco:
        tmp = tempfile.NamedTemporaryFile(suffix=".hsaco", delete=False)
        tmp.close()
        hsaco = tmp.name
    try:
        _, asm = compile_fn(cfg, hsaco)
        print(f"Config: {cfg.label}", file=out)
        print(asm, file=out)
        # what the descriptor says was selected: a mapping the pre-built kernels do not have is
        # recorded under the name of the kernel that runs instead
        result_label = None
        try:
            with open(hsaco) as f:
                desc = json.load(f)
            if desc.get("mapping_honoured") is False:
                result_label = desc["kernel"]
                print(f"Mapping not honoured ({', '.join(desc['mapping_not_honoured'])}): "
                      f"results are recorded as {result_label}", file=out)
        except (OSError, ValueError, KeyError):
            pass  # a compile_fn that writes a real code object
        if getattr(args, "compile_only", False):
            return None
        if not system_has_gpu("gfx950"):
            print("No GPUs detected -- skipping execution.", file=out)
            return None
        init_mode = getattr(args, "init", INIT_DEFAULT)
        A, B = make_inputs(cfg, init_mode)
        _, times_ns = execute_fn(cfg, hsaco, iterations, A, B, skip_gpu_check=True)
        measured = times_ns[WARMUP_ITERATIONS:]
        if not measured:
            print(f"\nNo measurements after warmup ({iterations} iterations), use a number > "
                  f"{WARMUP_ITERATIONS} e.g. --iterations=100", file=out)
            return None
        s = _compute_stats(measured, cfg.total_flops,
                           peak_tflops(cfg.mapping.mcpu, cfg.spec.dtype_ab))
        if s is None:
            print(f"\nInvalid timings (min={min(measured)} ns)", file=out)
            return None
        results_path = getattr(args, "results_file", None)
        if results_path:
            with open(results_path, "a") as rs:
                emit_one_result(rs, bench, cfg, s, label=result_label)
        print("\n--- Summary ---", file=out)
        print(f"  {'metric':<8s}  {'ms':>10s}  {'TFLOPS':>10s}  {'% peak':>8s}", file=out)
        for name, ms, tf, pct in (("p0", s.p0_ms, s.p0_tf, s.p0_pct), ("p10", s.p10_ms, s.p10_tf, None),
                                  ("p25", s.p25_ms, s.p25_tf, None), ("p50", s.p50_ms, s.p50_tf, s.p50_pct),
                                  ("p90", s.p90_ms, s.p90_tf, None), ("mean", s.mean_ms, s.mean_tf, s.mean_pct)):
            tail = f"{pct:>7.1f}%" if pct is not None else ""
            print(f"  {name:<8s}  {ms:>10.4f}  {tf:>10.1f}  {tail:>8s}", file=out)
        print(f"  {'stddev':<8s}  {'':>10s}  {s.stddev_tf:>10.1f}", file=out)

        print("\n--- Correctness check ---", file=out)
        expected = (_as_f32(A, cfg.spec.dtype_ab) @ _as_f32(B, cfg.spec.dtype_ab).T).flatten()
        C_output, _ = execute_fn(cfg, hsaco, 1, A, B, skip_gpu_check=True)
        got = _as_f32(C_output, cfg.spec.dtype_c)
        try:
            np.testing.assert_allclose(got, expected, rtol=1e-2, atol=1e-2)
            print("PASS", file=out)
        except AssertionError:
            print(f"FAIL: max_abs_diff={float(np.max(np.abs(got - expected))):.6g}", file=out)
        return s
    finally:
        if tmp is not None:
            import os

            try:
                os.unlink(tmp.name)
            except OSError:
                pass


def mapping_candidates(M: int, N: int, K: int, *, dtype_ab: str = "bf16", dtype_c: str = "bf16"):
    """The mappings a sweep over one problem tries: every workgroup tile / wave grid the pre-built
    stream kernels have, on every operand path, that divides the problem (the weak-scale rule of
    `make_instance`).  The reference enumerates a much larger grid of compiler knobs
    (bench_perf_102_gemm_python_multitile_g2s_directb_cdna4.py:170-290); here a mapping can only
    steer the tile, the wave grid and the operand path, and mappings that resolve to the same
    kernel are timed once."""
    from .gemm_config import OperandPath, make_instance

    out = []
    for (tile, waves) in (((256, 256), (2, 4)), ((256, 256), (2, 2)), ((128, 256), (1, 4)), ((128, 128), (2, 2))):
        if M % tile[0] or N % tile[1]:
            continue
        for path in (OperandPath.LDS, OperandPath.DIRECT_B, OperandPath.DIRECT_AB):
            if path == OperandPath.DIRECT_AB and dtype_ab not in ("bf16", "f16"):
                continue
            try:
                out.append(make_instance(M, N, K, dtype_ab=dtype_ab, dtype_c=dtype_c, wg_tile=tile,
                                         waves=waves, operand_path=path))
            except (AssertionError, ValueError):
                continue
    return out


def bench_perf_sweep(configs, compile_fn, execute_fn, repro_cmd_fn=None, *, mcpu: str = "gfx950",
                     bench: str = "unknown", iterations: Optional[int] = None,
                     init_mode=INIT_DEFAULT, results_file: Optional[str] = None,
                     best_known_file: Optional[str] = None, apply: bool = False, out=sys.stdout):
    """Every config of `configs` through compile (select) -> timed launches -> one
    `BENCH_RESULT_JSON:` line each, then the lines against the best-known registry
    (OK / IMPROVE / REGRESS per size; `apply` writes new winners back).  Same interface idea as
    the reference's `bench_perf_sweep_pipelined` (bench_harness.py:1271-1501: configs, compile_fn,
    repro_cmd_fn, bench label, iterations, results file) without its process pools: nothing is
    compiled at run time, so one process does the whole sweep.  Configs that select the same
    pre-built kernel for the same problem are timed once and listed as aliases.

    Returns (results, selected): results = [(cfg, PerfStats)] sorted by p50, selected =
    {"label|operand path": kernel name}."""
    import json as _json
    import os
    import tempfile

    from . import perf_registry as R
    from .execution import system_has_gpu

    iterations = iterations or NUM_ITERATIONS
    configs = list(configs)
    selected, groups, failed = {}, {}, []
    tmpdir = tempfile.mkdtemp(prefix="astergemm_sweep_")
    for cfg in configs:
        path = os.path.join(tmpdir, f"{len(selected)}.hsaco")
        try:
            compile_fn(cfg, path)
            with open(path) as f:
                desc = _json.load(f)
        except Exception as exc:  # a mapping no kernel takes: reported, the sweep goes on
            failed.append((cfg, f"compile: {str(exc).splitlines()[0][:200]}"))
            continue
        selected[f"{cfg.label}|{cfg.mapping.operand_path.value}"] = desc["kernel"]
        key = (desc["kernel"], tuple(cfg.spec.gemm_size))
        groups.setdefault(key, []).append((cfg, path, desc))
    print(f"Sweep: {len(configs)} configs -> {len(groups)} distinct kernels, "
          f"{len(failed)} refused, {iterations} iterations each", file=out)
    results = []
    have_gpu = system_has_gpu(mcpu)
    if not have_gpu:
        print("No GPUs detected -- execution skipped.", file=out)
    for (kernel, size), members in (groups.items() if have_gpu else ()):
        # the mapping the kernel honours stands for the group; the others ran the same code
        members.sort(key=lambda m: not m[2].get("mapping_honoured", False))
        cfg, path, desc = members[0]
        try:
            A, B = make_inputs(cfg, init_mode)
            _, times_ns = execute_fn(cfg, path, iterations, A, B, skip_gpu_check=True)
            s = _compute_stats(times_ns[WARMUP_ITERATIONS:], cfg.total_flops,
                               peak_tflops(cfg.mapping.mcpu, cfg.spec.dtype_ab))
            if s is None:
                raise RuntimeError("no valid timings")
        except Exception as exc:
            failed.append((cfg, f"exec: {str(exc).splitlines()[0][:200]}"))
            continue
        # the reference's labels do not name the operand path: a run on pre-shuffled B, like a
        # mapping that was not honoured, is recorded under the name of the kernel that ran
        plain = cfg.mapping.operand_path.value == "lds"
        label = cfg.label if desc.get("mapping_honoured", False) and plain else kernel
        results.append((cfg, s))
        if results_file:
            with open(results_file, "a") as rs:
                emit_one_result(rs, bench, cfg, s, label=label)
        aliases = [m[0].label for m in members[1:]]
        print(f"  {s.p50_tf:8.1f} TF p50 ({s.p50_pct:5.1f} % peak)  {kernel}  <- {label}"
              + (f"  (+{len(aliases)} mappings that select the same kernel)" if aliases else ""), file=out)
    results.sort(key=lambda r: -r[1].p50_tf)
    for cfg, why in failed:
        print(f"  FAILED {cfg.label}: {why}"
              + (f"   repro: {repro_cmd_fn(cfg)}" if repro_cmd_fn else ""), file=out)
    if results and results_file and best_known_file is not None:
        data = R.load(best_known_file) if os.path.exists(best_known_file) else {}
        with open(results_file) as f:
            records = [r for r in R.parse_jsonl_results(f) if r.key.bench == bench]
        rows = R.dashboard_rows(data, records, mcpu=mcpu, bench=bench)
        print(R.render(rows), file=out)
        print(R.summarize(rows, allow_missing=True)[0], file=out)
        if apply:
            n = R.update_top_n(data, records)
            R.save(data, best_known_file)
            print(f"{n} slot(s) updated in {best_known_file}", file=out)
    return results, selected


def main(argv=None) -> int:
    """`python -m aster_amd.bench_harness --m M --n N --k K [--dtype bf16] ...`: the one-command
    sweep over the mappings of one problem."""
    import argparse

    from . import gemm as AG
    from . import perf_registry as R

    ap = argparse.ArgumentParser(description="Sweep the mappings of one GEMM problem through the pre-built kernels")
    ap.add_argument("--m", type=int, required=True)
    ap.add_argument("--n", type=int, required=True)
    ap.add_argument("--k", type=int, required=True)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16"])
    ap.add_argument("--out-dtype", default="bf16", choices=["bf16", "f16", "f32"])
    ap.add_argument("--iterations", type=int, default=NUM_ITERATIONS)
    ap.add_argument("--results-file", default="sweep_results.jsonl")
    ap.add_argument("--best-known-file", default=R.DEFAULT_PATH)
    ap.add_argument("--apply", action="store_true", help="write new winners into the registry")
    args = ap.parse_args(argv)
    bench = f"astergemm_{args.dtype}"
    configs = mapping_candidates(args.m, args.n, args.k, dtype_ab=args.dtype, dtype_c=args.out_dtype)
    if not configs:
        print("no mapping divides this problem (M, N multiples of 128 are the smallest tile)")
        return 2
    results, _ = bench_perf_sweep(
        configs, AG.compile_gemm, AG.execute_gemm_hsaco,
        lambda cfg: f"python -m aster_amd.bench_harness --m {args.m} --n {args.n} --k {args.k}  # {cfg.label}",
        bench=bench, iterations=args.iterations, results_file=args.results_file,
        best_known_file=args.best_known_file, apply=args.apply)
    return 0 if results else 1


if __name__ == "__main__":
    sys.exit(main())
