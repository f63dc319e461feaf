"""The evaluation CLI end to end on the GPU: `--suite baseline --backend directory` scores every
operator correct and writes the four result files (BackendBench/output.py:116-196,236-288) in the
reference's schema, plus roofline_summary.csv for the timed cases whose work the suite declares."""

import csv
import json
import os

import pytest
from click.testing import CliRunner

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cli_baseline_suite_writes_result_files_with_roofline_columns(tmp_path):
    from backendbench_amd.scripts.main import cli

    print("CLI: --suite baseline --scale 0.05 --backend directory", flush=True)
    out = tmp_path / "run"
    res = CliRunner().invoke(cli, ["--suite", "baseline", "--scale", "0.05", "--backend", "directory",
                                   "--ops-directory", os.path.join(ROOT, "generated_kernels"), "--log-dir", str(out)],
                             catch_exceptions=False)
    assert res.exit_code == 0, res.output
    assert "correctness score (mean pass rate over all operators): 1.00" in res.output, res.output
    assert sorted(f.name for f in out.iterdir()) == ["OVERALL_SUMMARY.md", "failed_tests.json", "full_results.json",
                                                     "operator_summary.csv", "roofline_summary.csv"]
    assert json.loads((out / "failed_tests.json").read_text()) == []
    rows = {r["operator"]: r for r in csv.DictReader(open(out / "operator_summary.csv"))}
    assert len(rows) >= 28 + 26   # functional and out= overloads
    assert list(rows["add.Tensor"]) == ["operator", "total_tests", "correctness_tests", "performance_tests",
                                        "passed_correctness_tests", "passed_performance_tests", "failed_correctness_tests",
                                        "failed_performance_tests", "correctness_rate", "avg_speedup", "geomean_speedup",
                                        "max_absolute_error", "max_relative_error"]   # the reference's columns, no more
    roof = {}
    for r in csv.DictReader(open(out / "roofline_summary.csv")):
        roof.setdefault(r["operator"], r)                        # first row per operator = the case with the most work
    for op, bound, unit in [("add.Tensor", "hbm", "GB/s"), ("_softmax.default", "hbm", "GB/s"), ("mm.default", "mfma", "TFLOP/s"),
                            ("embedding.default", "hbm", "GB/s"), ("argmax.default", "hbm", "GB/s")]:
        assert float(rows[op]["correctness_rate"]) == 1.0, op
        r = roof[op]
        assert r["bound"] == bound and r["achieved_unit"] == unit, (op, r)
        assert float(r["algorithmic_work"]) > 0 and 0.0 < float(r["roofline_frac"]) < 1.0, (op, r)
        assert abs(float(r["achieved"]) - float(r["algorithmic_work"]) / (float(r["benchmark_time_ms"]) * 1e-3) / (1e9 if unit == "GB/s" else 1e12)) < 1e-3
    records = json.loads((out / "full_results.json").read_text())
    perf = [r for r in records if r["test_type"] == "performance" and r["op_name"] == "_softmax.default"]
    assert perf and perf[0]["successfully_ran"] and "bound" not in perf[0]
    text = (out / "OVERALL_SUMMARY.md").read_text()
    assert "# BackendBench Run Summary" in text and "| Correctness Score | 1.00 |" in text
