"""Result files of an evaluation run.

Writes the same four files, with the same fields in the same order, as
BackendBench/output.py:116-288: full_results.json (every test result, sorted by op then args),
operator_summary.csv (one row per operator), failed_tests.json and OVERALL_SUMMARY.md - a
consumer of the reference's schema reads them unchanged.  What this build measures beyond the
reference (algorithmic work of a timed case, GB/s or TFLOP/s, fraction of the MI355X peak) goes
to a fifth file of its own, roofline_summary.csv, written only when the suite declared the work
of some timed case.
"""

import csv
import json
import logging
from collections import defaultdict
from dataclasses import asdict
from pathlib import Path

import torch

from .eval import CorrectnessTestResult, PerformanceTestResult

logger = logging.getLogger(__name__)


def _geomean(xs):
    return torch.tensor(xs, dtype=torch.float64).log().mean().exp().item() if xs else 0.0


ROOFLINE_FIELDS = ("algorithmic_work", "bound", "achieved", "achieved_unit", "roofline_frac")


def _reference_record(result):
    """asdict() of a result with exactly the reference's fields (BackendBench/eval.py:24-46)."""
    rec = asdict(result)
    for name in ROOFLINE_FIELDS:
        rec.pop(name, None)
    return rec


def roofline_rows(performance_results):
    """One row per timed case whose suite declared its algorithmic work: what roofline_summary.csv holds."""
    rows = []
    for r in performance_results or []:
        if r.successfully_ran and getattr(r, "roofline_frac", None) is not None:
            rows.append({"operator": r.op_name, "args": r.args, "benchmark_time_ms": r.benchmark_time_ms,
                         "speedup": r.speedup, **{name: getattr(r, name) for name in ROOFLINE_FIELDS}})
    rows.sort(key=lambda row: (row["operator"], -row["algorithmic_work"], row["args"]))
    return rows


def prepare_results(correctness_results, performance_results):
    """(all results as dicts, failed tests as dicts, {op: summary row})."""
    order = lambda r: (r["op_name"], r["args"])
    all_results = sorted([_reference_record(r) for r in correctness_results] + [_reference_record(r) for r in performance_results], key=order)
    by_op = defaultdict(lambda: ([], []))
    for r in correctness_results:
        by_op[r.op_name][0].append(r)
    for r in performance_results:
        by_op[r.op_name][1].append(r)
    summaries = {}
    for op_name, (cs, ps) in by_op.items():
        passed_c = sum(1 for r in cs if r.is_correct)
        passed_p = sum(1 for r in ps if r.successfully_ran)
        errs = [(float(r.max_abs_error), float(r.max_rel_error)) for r in cs if r.max_abs_error and r.max_rel_error]
        speedups = [float(r.speedup) for r in ps if r.speedup]
        summaries[op_name] = {
            "operator": op_name,
            "total_tests": len(by_op),
            "correctness_tests": len(cs),
            "performance_tests": len(ps),
            "passed_correctness_tests": passed_c,
            "passed_performance_tests": passed_p,
            "failed_correctness_tests": len(cs) - passed_c,
            "failed_performance_tests": len(ps) - passed_p,
            "correctness_rate": passed_c / len(cs) if cs else 0.0,
            "avg_speedup": sum(speedups) / len(speedups) if speedups else 0.0,
            "geomean_speedup": _geomean(speedups),
            "max_absolute_error": max((e[0] for e in errs), default=0.0),
            "max_relative_error": max((e[1] for e in errs), default=0.0),
        }
    failed = sorted([_reference_record(r) for r in correctness_results if not r.is_correct]
                    + [_reference_record(r) for r in performance_results if not r.successfully_ran], key=order)
    return all_results, failed, summaries


def summary_rows(performance_results, correctness_results):
    """[(op, "xx.xxxx%", "y.yyyyx")] sorted by speed-up then correctness, descending; a
    performance test that did not run counts as speed-up 1.0."""
    correct, speed, names = defaultdict(list), defaultdict(list), set()
    for r in performance_results or []:
        speed[r.op_name].append(r.speedup if r.successfully_ran else 1.0)
        names.add(r.op_name)
    for r in correctness_results or []:
        correct[r.op_name].append(1.0 if r.is_correct else 0.0)
        names.add(r.op_name)
    rows = []
    for op in names:
        c = f"{sum(correct[op]) / len(correct[op]) * 100:.4f}%" if correct[op] else "N/A"
        s = f"{_geomean([float(x) for x in speed[op]]):.4f}x" if speed[op] else "N/A"
        rows.append((op, c, s))
    rows.sort(key=lambda row: (row[2], row[1]), reverse=True)
    return rows


def overall_summary_text(command, mean_correctness, geomean_perf, perf_at_p_score, p=1.0,
                         performance_results=None, correctness_results=None):
    lines = [
        "# BackendBench Run Summary\n", "## Command", "```bash", f"{command}", "```\n", "## Results\n",
        "| Metric | Value |", "|--------|-------|",
        f"| Correctness Score | {mean_correctness:.2f} |",
        f"| Performance Score (geomean speedup) | {geomean_perf:.2f} |",
        f"| Perf@{p} Score | {perf_at_p_score:.2f} |", "",
        "### Metric Descriptions\n",
        "- **Correctness Score**: Mean pass rate over all operators",
        "- **Performance Score**: Geometric mean speedup over all operators",
        f"- **Perf@{p} Score**: Rate of correct samples with a speedup greater than {p}", "",
        "## Output Files\n", "The following files are saved in this directory:\n",
        "- `full_results.json`: Complete test results for all operators",
        "- `operator_summary.csv`: Operator-level summary statistics",
        "- `failed_tests.json`: Log of failed tests (if any)",
        "- `OVERALL_SUMMARY.md`: This file",
        "### Operator Speedups vs Eager in Descending Order\n",
        "| Operator | Correctness Ratio | Speedup vs Eager |", "|----------|-----------|----------------|",
    ]
    lines += [f"| {op} | {c} | {s}|" for op, c, s in summary_rows(performance_results, correctness_results)]
    lines.append("")
    return "\n".join(lines)


def save_results(correctness_results, performance_results, output_path, command=None, mean_correctness=None,
                 geomean_perf=None, perf_at_p_score=None, p=1.0):
    base = Path(output_path)
    base.mkdir(parents=True, exist_ok=True)
    all_results, failed, summaries = prepare_results(correctness_results, performance_results)
    (base / "full_results.json").write_text(json.dumps(all_results, indent=2))
    if summaries:
        rows = list(summaries.values())
        with open(base / "operator_summary.csv", "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
            w.writeheader()
            w.writerows(rows)
    (base / "failed_tests.json").write_text(json.dumps(failed, indent=2))
    roof = roofline_rows(performance_results)
    if roof:
        with open(base / "roofline_summary.csv", "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(roof[0].keys()))
            w.writeheader()
            w.writerows(roof)
    if all(x is not None for x in (command, mean_correctness, geomean_perf, perf_at_p_score)):
        (base / "OVERALL_SUMMARY.md").write_text(
            overall_summary_text(command, mean_correctness, geomean_perf, perf_at_p_score, p,
                                 performance_results, correctness_results))
    print(f"Results saved to directory: {base.absolute()}")
    print(f"Overall summary saved to: {base.absolute()}/OVERALL_SUMMARY.md")
    return all_results, failed, summaries
