"""A measured run taken through the best-known registry and the regression dashboard on the GPU:
`run_single` timing -> `BENCH_RESULT_JSON:` line -> merge into a registry -> dashboard status.

The flow follows the reference's tools: result lines
(contrib/kittens/test/bench/tools/perf_bench_results_io.py:113-144), top-N update
(perf_best_known.py:9-68) and REGRESS / IMPROVE / OK margins (perf_dashboard.py:59-67).
"""
import argparse
import io
import json

import pytest

from aster_amd import bench_harness as BH, gemm as AG, perf_registry as R
from aster_amd.gemm_config import make_instance

pytestmark = pytest.mark.gpu


def _measure(cfg, results_file, bench="astergemm_bf16"):
    out = io.StringIO()
    args = argparse.Namespace(iterations=60, results_file=str(results_file))
    stats = BH.run_single(cfg, AG.compile_gemm, args, AG.execute_gemm_hsaco, bench=bench, out=out)
    text = out.getvalue()
    assert stats is not None and "PASS" in text, text
    return stats, text


def test_measured_run_through_registry_and_dashboard(gpu, tmp_path):
    results = tmp_path / "results.jsonl"
    registry = tmp_path / "best_known.json"
    cfg = make_instance(1024, 1024, 1024)            # the library's own 256 x 256, 2 x 4 geometry
    stats, _ = _measure(cfg, results)
    records = list(R.parse_jsonl_results(open(results)))
    assert len(records) == 1
    rec = records[0]
    assert rec.key == R.EntryKey("gfx950", "astergemm_bf16", 1024, 1024, 1024)
    assert rec.label == cfg.label and rec.tflops_median == pytest.approx(stats.p50_tf)
    assert 10.0 < rec.tflops_median < 2500.0
    # merge into an empty registry, then the same measurement reads OK against it
    data = {}
    assert R.update_top_n(data, records) == 1
    R.save(data, str(registry))
    data = R.load(str(registry))
    assert R.best_known(data, "gfx950", "astergemm_bf16", 1024, 1024, 1024) == cfg.label
    rows = R.dashboard_rows(data, records)
    assert [r.status for r in rows] == ["OK"]
    assert R.summarize(rows)[1] == 0
    # against an entry that expects 20 % less the run is an IMPROVE, 20 % more a REGRESS
    slot = data["gfx950"]["astergemm_bf16"][R.size_key(1024, 1024, 1024)]
    slot[0]["expected_tflops"] = rec.tflops_median / 1.2
    assert [r.status for r in R.dashboard_rows(data, records)] == ["IMPROVE"]
    slot[0]["expected_tflops"] = rec.tflops_median * 1.2
    rows = R.dashboard_rows(data, records)
    assert [r.status for r in rows] == ["REGRESS"] and R.summarize(rows)[1] == 1
    # the command-line form on the files, with a second measured run appended
    _measure(cfg, results)
    assert len(list(R.parse_jsonl_results(open(results)))) == 2
    R.save({}, str(registry))
    assert R.main(["--measurements", str(results), "--best-known-file", str(registry), "--apply"]) == 0
    assert R.main(["--measurements", str(results), "--best-known-file", str(registry)]) == 0


def test_unhonoured_mapping_is_recorded_under_the_kernel_that_ran(gpu, tmp_path):
    results = tmp_path / "results.jsonl"
    # the reference's best label geometry: 128 x 256 tile, 1 x 4 waves -- not a pre-built kernel
    cfg = make_instance(1024, 1024, 512, wg_tile=(128, 256), waves=(1, 4), pipeline_strategy=11)
    _, text = _measure(cfg, results)
    assert "Mapping not honoured" in text
    rec = next(R.parse_jsonl_results(open(results)))
    desc_kernel = AG.select_for_instance(cfg)[1].name.decode()
    assert rec.label == desc_kernel != cfg.label


def test_one_command_sweep_over_mappings(gpu, tmp_path):
    """Mappings of one problem -> select -> timed launches -> result lines -> registry, the shape
    of the reference's `bench_perf_sweep_pipelined` (bench_harness.py:1271-1501) in one process:
    mappings that select the same kernel are timed once, every timed kernel leaves a result line,
    and `--apply` puts the fastest into the registry, which the next run reads as OK."""
    results = tmp_path / "sweep.jsonl"
    registry = tmp_path / "best_known.json"
    argv = ["--m", "1024", "--n", "1024", "--k", "2048", "--iterations", "40",
            "--results-file", str(results), "--best-known-file", str(registry)]
    assert BH.main(argv + ["--apply"]) == 0
    records = list(R.parse_jsonl_results(open(results)))
    cfgs = BH.mapping_candidates(1024, 1024, 2048)
    kernels = {AG.select_for_instance(c)[1].name.decode() for c in cfgs}
    assert len(records) == len(kernels) >= 4          # 256x256 (2x4, 2x2), 128x256, 128x128, two paths
    assert len({r.label for r in records}) == len(records)
    assert all(10.0 < r.tflops_median < 2500.0 for r in records)
    data = R.load(str(registry))
    best = R.best_known(data, "gfx950", "astergemm_bf16", 1024, 1024, 2048)
    assert best == max(records, key=lambda r: r.tflops_median).label
    # the same measurements against the registry they produced: nothing regresses
    assert R.main(["--measurements", str(results), "--best-known-file", str(registry)]) == 0
