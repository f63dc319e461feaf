"""The evaluation CLI end to end on the GPU: `--suite baseline --backend directory` scores every
operator correct and writes the four result files (BackendBench/output.py:116-196,236-288) with
the roofline columns this build adds for timed cases whose work the suite declares."""

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
                                                     "operator_summary.csv"]
    assert json.loads((out / "failed_tests.json").read_text()) == []
    rows = {r["operator"]: r for r in csv.DictReader(open(out / "operator_summary.csv"))}
    assert len(rows) >= 28
    for name in ("operator", "correctness_rate", "geomean_speedup", "algorithmic_work", "bound", "achieved",
                 "achieved_unit", "roofline_frac"):
        assert name in rows["add.Tensor"], name
    for op, bound, unit in [("add.Tensor", "hbm", "GB/s"), ("_softmax.default", "hbm", "GB/s"), ("mm.default", "mfma", "TFLOP/s"),
                            ("embedding.default", "hbm", "GB/s"), ("argmax.default", "hbm", "GB/s")]:
        r = rows[op]
        assert float(r["correctness_rate"]) == 1.0, op
        assert r["bound"] == bound and r["achieved_unit"] == unit, (op, r)
        assert float(r["algorithmic_work"]) > 0 and 0.0 < float(r["roofline_frac"]) < 1.0, (op, r)
    records = json.loads((out / "full_results.json").read_text())
    perf = [r for r in records if r["test_type"] == "performance" and r["op_name"] == "_softmax.default"]
    assert perf and perf[0]["successfully_ran"] and perf[0]["bound"] == "hbm"
    assert abs(perf[0]["achieved"] - perf[0]["algorithmic_work"] / (perf[0]["benchmark_time_ms"] * 1e-3) / 1e9) < 1e-6
    text = (out / "OVERALL_SUMMARY.md").read_text()
    assert "# BackendBench Run Summary" in text and "| Correctness Score | 1.00 |" in text
