"""Result files: names, fields and summary rows (reference: BackendBench/output.py:116-288,
expectations in test/test_output.py:116-172)."""

import csv
import json

from backendbench_amd.eval import CorrectnessTestResult, PerformanceTestResult
from backendbench_amd.output import overall_summary_text, prepare_results, roofline_rows, save_results, summary_rows


def results():
    c = [CorrectnessTestResult("add.Tensor", "a1", True, max_abs_error=0.5, max_rel_error=0.25),
         CorrectnessTestResult("add.Tensor", "a0", False, error_msg="bad", max_abs_error=2.0, max_rel_error=1.0),
         CorrectnessTestResult("relu.default", "r0", True, max_abs_error=0.0, max_rel_error=0.0)]
    p = [PerformanceTestResult("add.Tensor", "a1", 2.0, 1.0, 2.0, successfully_ran=True),
         PerformanceTestResult("add.Tensor", "a0", 8.0, 1.0, 8.0, successfully_ran=True),
         PerformanceTestResult("relu.default", "r0", None, None, 3.0, error_msg="x", successfully_ran=False)]
    return c, p


def test_prepare_results():
    c, p = results()
    everything, failed, summary = prepare_results(c, p)
    assert [r["args"] for r in everything] == ["a0", "a0", "a1", "a1", "r0", "r0"]
    assert [(r["op_name"], r["test_type"]) for r in failed] == [("add.Tensor", "correctness"), ("relu.default", "performance")]
    s = summary["add.Tensor"]
    assert s["correctness_tests"] == 2 and s["passed_correctness_tests"] == 1 and s["failed_correctness_tests"] == 1
    assert s["correctness_rate"] == 0.5 and s["avg_speedup"] == 5.0 and abs(s["geomean_speedup"] - 4.0) < 1e-9
    assert s["max_absolute_error"] == 2.0 and s["max_relative_error"] == 1.0
    assert summary["relu.default"]["passed_performance_tests"] == 0 and summary["relu.default"]["geomean_speedup"] == 0.0
    assert list(s) == ["operator", "total_tests", "correctness_tests", "performance_tests", "passed_correctness_tests",
                       "passed_performance_tests", "failed_correctness_tests", "failed_performance_tests",
                       "correctness_rate", "avg_speedup", "geomean_speedup", "max_absolute_error", "max_relative_error"]
    # exactly the reference's record fields (BackendBench/eval.py:24-46), nothing of this build's on top
    perf = [r for r in everything if r["test_type"] == "performance"][0]
    assert list(perf) == ["op_name", "args", "speedup", "benchmark_time_ms", "reference_time_ms", "error_msg",
                          "successfully_ran", "test_type"]
    corr = [r for r in everything if r["test_type"] == "correctness"][0]
    assert list(corr) == ["op_name", "args", "is_correct", "error_msg", "error_type", "traceback", "max_abs_error",
                          "max_rel_error", "test_type"]


def test_roofline_columns():
    """Records of timed cases whose suite declares their algorithmic work carry GB/s or TFLOP/s and the
    fraction of the MI355X peak; the operator row takes the case with the most work."""
    from types import SimpleNamespace

    from backendbench_amd.eval import roofline_columns

    hbm = SimpleNamespace(case=SimpleNamespace(work=134217728.0, bound="hbm"))
    cols = roofline_columns(hbm, 0.024, True)
    assert cols["achieved_unit"] == "GB/s" and abs(cols["achieved"] - 134217728 / 0.024e-3 / 1e9) < 1e-6
    assert abs(cols["roofline_frac"] - cols["achieved"] / 8000.0) < 1e-12
    mfma = SimpleNamespace(case=SimpleNamespace(work=369367187456.0, bound="mfma"))
    cols = roofline_columns(mfma, 0.25, True)
    assert cols["achieved_unit"] == "TFLOP/s" and abs(cols["achieved"] - 1477.468749824) < 1e-6
    assert abs(cols["roofline_frac"] - 1477.468749824 / 2500.0) < 1e-9
    assert roofline_columns(hbm, 0.024, False) == {}           # CPU timings (seconds, not a GPU rate)
    assert roofline_columns(SimpleNamespace(), 0.024, True) == {}
    p = [PerformanceTestResult("mm.default", "small", 1.5, 0.01, 0.015, successfully_ran=True,
                               **roofline_columns(SimpleNamespace(case=SimpleNamespace(work=1e9, bound="mfma")), 0.01, True)),
         PerformanceTestResult("mm.default", "big", 1.2, 0.25, 0.3, successfully_ran=True, **cols)]
    everything, _, summary = prepare_results([], p)
    assert "roofline_frac" not in summary["mm.default"] and all("bound" not in r for r in everything)
    rows = roofline_rows(p)                                      # the fifth file: the case with the most work first
    assert [r["args"] for r in rows] == ["big", "small"] and rows[0]["operator"] == "mm.default"
    assert rows[0]["algorithmic_work"] == 369367187456.0 and rows[0]["bound"] == "mfma" and rows[0]["achieved_unit"] == "TFLOP/s"
    assert abs(rows[0]["roofline_frac"] - 0.5909874999296) < 1e-9
    assert roofline_rows(results()[1]) == []                     # no declared work: no rows, no file


def test_summary_rows_and_text():
    c, p = results()
    rows = summary_rows(p, c)
    assert rows == [("add.Tensor", "50.0000%", "4.0000x"), ("relu.default", "100.0000%", "1.0000x")]
    text = overall_summary_text("cmd --x", 0.5, 2.0, 0.25, 1.0, p, c)
    assert "# BackendBench Run Summary" in text and "| Correctness Score | 0.50 |" in text
    assert "| Perf@1.0 Score | 0.25 |" in text and "| add.Tensor | 50.0000% | 4.0000x|" in text


def test_save_results_writes_four_files(tmp_path):
    c, p = results()
    save_results(c, p, str(tmp_path / "out"), command="cmd", mean_correctness=0.5, geomean_perf=2.0, perf_at_p_score=0.25)
    names = sorted(f.name for f in (tmp_path / "out").iterdir())
    assert names == ["OVERALL_SUMMARY.md", "failed_tests.json", "full_results.json", "operator_summary.csv"]
    assert len(json.loads((tmp_path / "out" / "full_results.json").read_text())) == 6
    rows = list(csv.DictReader(open(tmp_path / "out" / "operator_summary.csv")))
    assert {r["operator"] for r in rows} == {"add.Tensor", "relu.default"}
    save_results(c, p, str(tmp_path / "bare"))
    assert not (tmp_path / "bare" / "OVERALL_SUMMARY.md").exists()
    from types import SimpleNamespace

    from backendbench_amd.eval import roofline_columns

    cols = roofline_columns(SimpleNamespace(case=SimpleNamespace(work=134217728.0, bound="hbm")), 0.024, True)
    p2 = p + [PerformanceTestResult("_softmax.default", "s0", 1.3, 0.024, 0.031, successfully_ran=True, **cols)]
    save_results(c, p2, str(tmp_path / "roof"))
    rows = list(csv.DictReader(open(tmp_path / "roof" / "roofline_summary.csv")))
    assert len(rows) == 1 and rows[0]["operator"] == "_softmax.default" and rows[0]["bound"] == "hbm"
    assert abs(float(rows[0]["roofline_frac"]) - 134217728 / 0.024e-3 / 1e9 / 8000.0) < 1e-9
