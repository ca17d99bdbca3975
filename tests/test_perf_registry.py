"""Best-known registry and regression dashboard (host logic, no GPU).

Behaviour pinned to the reference's tools: BENCH_RESULT_JSON parsing and max-merge
(contrib/kittens/test/bench/tools/perf_bench_results_io.py:46-110), registry shape and top-5
slots (perf_best_known.py:9-68), dashboard statuses and exit codes
(perf_dashboard.py:38-63, 118-134)."""
import io
import json
import os

import pytest

from aster_amd import perf_registry as R

LINE = R.RESULT_SENTINEL + json.dumps({
    "mcpu": "gfx950", "bench": "astergemm_bf16", "M": 8192, "N": 8192, "K": 8192,
    "label": "stream_bf16_256x256_w2x4_bf16", "tflops_median": 1512.3, "tflops_p10": 1490.0,
    "tflops_p90": "n/a", "sample_n": 1})


def rec(label, tf, bench="astergemm_bf16", size=(8192, 8192, 8192)):
    return R.BenchResultRecord(R.EntryKey("gfx950", bench, *size), label, tf)


def test_parse_skips_noise_and_malformed_lines():
    lines = ["hello", "x " + LINE + "\n", R.RESULT_SENTINEL + "{not json",
             R.RESULT_SENTINEL + json.dumps({"mcpu": "gfx950"}),                     # missing keys
             R.RESULT_SENTINEL + json.dumps({"mcpu": "g", "bench": "b", "M": "x", "N": 1, "K": 1,
                                             "label": "l", "tflops_median": 1})]     # bad int
    out = list(R.parse_jsonl_results(lines))
    assert len(out) == 1
    r = out[0]
    assert r.key == R.EntryKey("gfx950", "astergemm_bf16", 8192, 8192, 8192)
    assert r.tflops_median == 1512.3 and r.tflops_p10 == 1490.0 and r.tflops_p90 is None
    assert r.tflops_mean is None and r.sample_n == 1


def test_max_merge():
    rs = [rec("a", 10), rec("a", 12), rec("b", 11), rec("a", 5, size=(1, 2, 3))]
    kl = R.max_merge_by_key_label(rs)
    assert kl[(rs[0].key, "a")].tflops_median == 12 and len(kl) == 3
    k = R.max_merge_by_key(rs)
    assert k[rs[0].key].label == "a" and k[rs[3].key].tflops_median == 5


def test_size_key_roundtrip_and_lookup():
    assert R.parse_size_key(R.size_key(4096, 14336, 4096)) == (4096, 14336, 4096)
    data = R.load()
    assert R.best_known(data, "gfx950", "astergemm_bf16", 8192, 8192, 8192) == \
        "stream_bf16_256x256_w2x4_bf16"
    assert R.best_known(data, "gfx950", "astergemm_bf16", 1, 1, 1) is None
    # every slot is sorted best first and holds at most TOP_N entries
    for _, _, _, slot in R.iter_registry(data):
        vals = [e["expected_tflops"] for e in slot]
        assert vals == sorted(vals, reverse=True) and len(slot) <= R.TOP_N


@pytest.mark.parametrize("measured,status", [(None, "MISS"), (94.9, "REGRESS"), (95.0, "OK"),
                                             (103.0, "OK"), (103.1, "IMPROVE")])
def test_status_margins(measured, status):
    assert R.status_of(measured, 100.0) == status


def test_dashboard_rows_and_exit_codes():
    data = {"gfx950": {"b": {"8x8x8": [{"label": "x", "expected_tflops": 100.0},
                                       {"label": "y", "expected_tflops": 90.0}]}}}
    k = dict(bench="b", size=(8, 8, 8))
    rows = R.dashboard_rows(data, [rec("x", 80.0, **k), rec("y", 91.0, **k)])
    assert [(r.label, r.status) for r in rows] == [("x", "REGRESS"), ("y", "OK")]
    assert R.summarize(rows)[1] == 1
    rows = R.dashboard_rows(data, [rec("x", 120.0, **k)])
    assert {r.label: r.status for r in rows} == {"x": "IMPROVE", "y": "MISS"}
    assert R.summarize(rows)[1] == 2 and R.summarize(rows, allow_missing=True)[1] == 0
    rows = R.dashboard_rows(data, [rec("x", 100.0, **k), rec("y", 90.0, **k)])
    assert R.summarize(rows)[1] == 0
    assert "REGRESS" not in R.render(rows) and "delta_pct" in R.render(rows)


def test_update_top_n_keeps_five_best_one_per_label():
    data = {}
    rs = [rec(f"l{i}", 100.0 + i) for i in range(7)] + [rec("l3", 200.0), rec("l6", 1.0)]
    assert R.update_top_n(data, rs) == 1
    slot = data["gfx950"]["astergemm_bf16"]["8192x8192x8192"]
    assert [e["label"] for e in slot] == ["l3", "l6", "l5", "l4", "l2"]
    assert slot[0]["expected_tflops"] == 200.0
    assert R.update_top_n(data, rs) == 0                     # idempotent
    assert R.update_top_n(data, [rec("l0", 50.0)]) == 0      # worse than everything stored


def test_cli_apply_writes_registry(tmp_path, capsys):
    reg = tmp_path / "bk.json"
    reg.write_text(json.dumps({"gfx950": {"astergemm_bf16": {"8192x8192x8192": [
        {"label": "stream_bf16_256x256_w2x4_bf16", "expected_tflops": 1400.0}]}}}))
    meas = tmp_path / "run.jsonl"
    meas.write_text(LINE + "\n")
    code = R.main(["--measurements", str(meas), "--best-known-file", str(reg), "--apply"])
    out = capsys.readouterr().out
    assert code == 0 and "IMPROVE" in out and "1 slot(s) updated" in out
    assert json.loads(reg.read_text())["gfx950"]["astergemm_bf16"]["8192x8192x8192"][0][
        "expected_tflops"] == 1512.3


def test_harness_emits_lines_the_registry_parses():
    from aster_amd import bench_harness as H
    from aster_amd.gemm_config import make_instance
    cfg = make_instance(256, 256, 256)
    stats = H._compute_stats([1000, 1100, 1200, 900], cfg.spec.total_flops, 2500.0)
    buf = io.StringIO()
    H.emit_one_result(buf, "astergemm_f16", cfg, stats)
    (r,) = list(R.parse_jsonl_results(buf.getvalue().splitlines()))
    assert r.key == R.EntryKey(cfg.mapping.mcpu, "astergemm_f16", 256, 256, 256)
    assert r.label == cfg.label and r.tflops_median == pytest.approx(stats.p50_tf)
