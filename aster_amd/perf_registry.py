"""Best-known registry and regression check for measured GEMM kernels.

Counterpart of the reference's bench tools
(contrib/kittens/test/bench/tools/perf_bench_results_io.py:16-144,
perf_best_known.py:23-68, perf_best_known_update.py, perf_dashboard.py:38-63):

* a measurement is one `BENCH_RESULT_JSON:{...}` line keyed by
  (mcpu, bench, M, N, K) and a config label; several runs are max-merged;
* the registry is `{mcpu: {bench: {"MxNxK": [{label, expected_tflops}, ...]}}}`,
  every size slot holding its top five labels, best first;
* the dashboard compares measurements with the stored entries label by label:
  REGRESS below expected * (1 - 0.05), IMPROVE above expected * (1 + 0.03),
  OK otherwise, MISS when a stored entry was not measured; exit code 1 on any
  REGRESS, else 2 on any MISS (unless allowed), else 0.

`python -m aster_amd.perf_registry --measurements run.jsonl [--best-known-file F]
[--apply]` prints the table; `--apply` writes new winners back.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from dataclasses import dataclass
from typing import Dict, Iterable, Iterator, List, Optional, Tuple

RESULT_SENTINEL = "BENCH_RESULT_JSON:"
TOP_N = 5
DEFAULT_IMPROVE_MARGIN = 0.03
DEFAULT_REGRESS_MARGIN = 0.05
DEFAULT_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "best_known.json")
_STATUS_RANK = {"REGRESS": 0, "MISS": 1, "IMPROVE": 2, "OK": 3}


@dataclass(frozen=True)
class EntryKey:
    """Identity of a (problem, target) measurement slot."""
    mcpu: str
    bench: str
    M: int
    N: int
    K: int


@dataclass(frozen=True)
class BenchResultRecord:
    """One measured config from one run; `tflops_median` is the headline."""
    key: EntryKey
    label: str
    tflops_median: float
    tflops_p10: Optional[float] = None
    tflops_p90: Optional[float] = None
    tflops_mean: Optional[float] = None
    sample_n: int = 1


def _opt_float(v) -> Optional[float]:
    try:
        return None if v is None else float(v)
    except (TypeError, ValueError):
        return None


def parse_jsonl_results(stream: Iterable[str]) -> Iterator[BenchResultRecord]:
    """One record per well-formed BENCH_RESULT_JSON line; everything else is skipped."""
    for raw in stream:
        at = raw.find(RESULT_SENTINEL)
        if at < 0:
            continue
        try:
            d = json.loads(raw[at + len(RESULT_SENTINEL):].strip())
            key = EntryKey(d["mcpu"], d["bench"], int(d["M"]), int(d["N"]), int(d["K"]))
            label, median = d["label"], float(d["tflops_median"])
        except (json.JSONDecodeError, KeyError, TypeError, ValueError):
            continue
        yield BenchResultRecord(key, label, median, _opt_float(d.get("tflops_p10")),
                                _opt_float(d.get("tflops_p90")), _opt_float(d.get("tflops_mean")),
                                int(d.get("sample_n", 1)))


def max_merge_by_key_label(records: Iterable[BenchResultRecord]
                           ) -> Dict[Tuple[EntryKey, str], BenchResultRecord]:
    """Best record (highest median) per (key, label) across runs."""
    best: Dict[Tuple[EntryKey, str], BenchResultRecord] = {}
    for r in records:
        slot = (r.key, r.label)
        if slot not in best or r.tflops_median > best[slot].tflops_median:
            best[slot] = r
    return best


def max_merge_by_key(records: Iterable[BenchResultRecord]) -> Dict[EntryKey, BenchResultRecord]:
    """Best record per key across runs and labels."""
    best: Dict[EntryKey, BenchResultRecord] = {}
    for (key, _), r in max_merge_by_key_label(records).items():
        if key not in best or r.tflops_median > best[key].tflops_median:
            best[key] = r
    return best


# ---- registry ---------------------------------------------------------------------------

def size_key(M: int, N: int, K: int) -> str:
    return f"{M}x{N}x{K}"


def parse_size_key(key: str) -> Tuple[int, int, int]:
    m, n, k = key.split("x")
    return int(m), int(n), int(k)


def load(path: str = DEFAULT_PATH) -> dict:
    with open(path) as f:
        return json.load(f)


def save(data: dict, path: str = DEFAULT_PATH) -> None:
    tmp = str(path) + ".tmp"
    with open(tmp, "w") as f:
        json.dump(data, f, indent=2, sort_keys=True)
        f.write("\n")
    os.replace(tmp, path)


def best_known_top_n(data: dict, mcpu: str, bench: str, M: int, N: int, K: int) -> List[dict]:
    return list(data.get(mcpu, {}).get(bench, {}).get(size_key(M, N, K)) or [])


def best_known(data: dict, mcpu: str, bench: str, M: int, N: int, K: int) -> Optional[str]:
    slot = best_known_top_n(data, mcpu, bench, M, N, K)
    return slot[0]["label"] if slot else None


def iter_registry(data: dict, mcpu_filter: Optional[str] = None, bench_filter: Optional[str] = None):
    for mcpu in sorted(data):
        if mcpu_filter and mcpu != mcpu_filter:
            continue
        for bench in sorted(data[mcpu]):
            if bench_filter and bench != bench_filter:
                continue
            for sk in sorted(data[mcpu][bench], key=parse_size_key):
                yield mcpu, bench, sk, data[mcpu][bench][sk]


def update_top_n(data: dict, records: Iterable[BenchResultRecord], top_n: int = TOP_N) -> int:
    """Merge measurements into the registry: per size slot keep the `top_n` best labels, one
    entry per label (its best median, rounded to 0.1).  Returns the number of slots changed."""
    changed = 0
    merged = max_merge_by_key_label(records)
    by_key: Dict[EntryKey, List[BenchResultRecord]] = {}
    for (key, _), r in merged.items():
        by_key.setdefault(key, []).append(r)
    for key, recs in by_key.items():
        slot_map = data.setdefault(key.mcpu, {}).setdefault(key.bench, {})
        sk = size_key(key.M, key.N, key.K)
        old = list(slot_map.get(sk) or [])
        best = {e["label"]: float(e["expected_tflops"]) for e in old}
        for r in recs:
            v = round(r.tflops_median, 1)
            if v > best.get(r.label, float("-inf")):
                best[r.label] = v
        new = [{"expected_tflops": v, "label": l}
               for l, v in sorted(best.items(), key=lambda kv: (-kv[1], kv[0]))[:top_n]]
        if new != old:
            slot_map[sk] = new
            changed += 1
    return changed


# ---- dashboard --------------------------------------------------------------------------

@dataclass
class Row:
    key: EntryKey
    rank: int
    label: str
    expected_tflops: float
    measured: Optional[float]
    status: str


def status_of(measured: Optional[float], expected: float,
              regress_margin: float = DEFAULT_REGRESS_MARGIN,
              improve_margin: float = DEFAULT_IMPROVE_MARGIN) -> str:
    if measured is None:
        return "MISS"
    if measured < expected * (1.0 - regress_margin):
        return "REGRESS"
    if measured > expected * (1.0 + improve_margin):
        return "IMPROVE"
    return "OK"


def dashboard_rows(data: dict, records: Iterable[BenchResultRecord], *,
                   mcpu: Optional[str] = None, bench: Optional[str] = None,
                   regress_margin: float = DEFAULT_REGRESS_MARGIN,
                   improve_margin: float = DEFAULT_IMPROVE_MARGIN) -> List[Row]:
    measured = {k: r.tflops_median for k, r in max_merge_by_key_label(records).items()}
    rows: List[Row] = []
    for m, b, sk, slot in iter_registry(data, mcpu, bench):
        M, N, K = parse_size_key(sk)
        key = EntryKey(m, b, M, N, K)
        for rank, entry in enumerate(slot or [], start=1):
            got = measured.get((key, entry["label"]))
            rows.append(Row(key, rank, entry["label"], float(entry["expected_tflops"]), got,
                            status_of(got, float(entry["expected_tflops"]), regress_margin,
                                      improve_margin)))
    rows.sort(key=lambda r: (_STATUS_RANK[r.status], r.key.mcpu, r.key.bench, r.key.M, r.key.N,
                             r.key.K, r.rank))
    return rows


def summarize(rows: List[Row], allow_missing: bool = False) -> Tuple[str, int]:
    counts = {s: sum(1 for r in rows if r.status == s) for s in _STATUS_RANK}
    slots = len({r.key for r in rows})
    text = (f"{len(rows)} stored entries across {slots} (mcpu,bench,M,N,K) slot(s) checked.  "
            f"{counts['REGRESS']} REGRESS, {counts['IMPROVE']} IMPROVE, {counts['OK']} OK"
            + (f", {counts['MISS']} MISS" if counts["MISS"] else "") + ".")
    code = 1 if counts["REGRESS"] else (2 if counts["MISS"] and not allow_missing else 0)
    return text, code


def render(rows: List[Row]) -> str:
    head = ["mcpu", "bench", "M", "N", "K", "rank", "expected", "measured", "delta_pct", "status", "label"]
    body = []
    for r in rows:
        delta = "---" if r.measured is None or r.expected_tflops == 0 else \
            f"{(r.measured - r.expected_tflops) / r.expected_tflops * 100.0:+.2f}%"
        body.append([r.key.mcpu, r.key.bench, str(r.key.M), str(r.key.N), str(r.key.K), f"#{r.rank}",
                     f"{r.expected_tflops:.1f}", "---" if r.measured is None else f"{r.measured:.1f}",
                     delta, r.status, r.label])
    widths = [max(len(h), *(len(row[i]) for row in body)) if body else len(h)
              for i, h in enumerate(head)]
    fmt = "  ".join("{:<" + str(w) + "}" for w in widths)
    return "\n".join([fmt.format(*head), fmt.format(*("-" * w for w in widths))]
                     + [fmt.format(*row) for row in body])


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(description="Compare BENCH_RESULT_JSON lines with the registry")
    ap.add_argument("--measurements", required=True, help="file of BENCH_RESULT_JSON lines, '-' = stdin")
    ap.add_argument("--best-known-file", default=DEFAULT_PATH)
    ap.add_argument("--mcpu", default=None)
    ap.add_argument("--bench", default=None)
    ap.add_argument("--regress-margin", type=float, default=DEFAULT_REGRESS_MARGIN)
    ap.add_argument("--improve-margin", type=float, default=DEFAULT_IMPROVE_MARGIN)
    ap.add_argument("--allow-missing", action="store_true")
    ap.add_argument("--apply", action="store_true", help="write new winners into the registry")
    args = ap.parse_args(argv)
    data = load(args.best_known_file)
    stream = sys.stdin if args.measurements == "-" else open(args.measurements)
    try:
        records = list(parse_jsonl_results(stream))
    finally:
        if stream is not sys.stdin:
            stream.close()
    rows = dashboard_rows(data, records, mcpu=args.mcpu, bench=args.bench,
                          regress_margin=args.regress_margin, improve_margin=args.improve_margin)
    print(render(rows))
    text, code = summarize(rows, args.allow_missing)
    print("\n" + text)
    if args.apply:
        n = update_top_n(data, records)
        save(data, args.best_known_file)
        print(f"{n} slot(s) updated in {args.best_known_file}")
    return code


if __name__ == "__main__":
    sys.exit(main())
