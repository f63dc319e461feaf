"""Evaluator semantics: tolerance, nesting, timing recipe, scores.  Expectations follow the
reference's tests (test/test_eval.py:43-94, 168-180, 209-253; test/test_smoke.py:43-54)."""

import numpy as np
import pytest
import torch

from backendbench_amd import eval as ev
from backendbench_amd.backends import AtenBackend
from backendbench_amd.suite import SmokeTestSuite
from backendbench_amd.suite.base import Test as Case


def test_allclose_tolerance():
    assert ev.allclose(torch.tensor([3.0]), torch.tensor([3.01]))          # inside 1e-2 + 1e-2*3
    assert not ev.allclose(torch.tensor([3.0]), torch.tensor([3.1]))
    assert not ev.allclose(torch.tensor([3.0]), torch.tensor([2.9]))
    nan = torch.tensor([float("nan"), 1.0])
    assert ev.allclose(nan, nan.clone())
    assert not ev.allclose(torch.tensor([1.0]), torch.tensor([1.0], dtype=torch.float64))  # dtype is checked
    assert not ev.allclose(torch.zeros(2), torch.zeros(3))


def test_allclose_nested_and_scalars():
    a = (torch.ones(2), [torch.zeros(3), 5], "x")
    assert ev.allclose(a, (torch.ones(2), [torch.zeros(3), 5], "x"))
    assert not ev.allclose(a, (torch.ones(2), [torch.zeros(3), 6], "x"))
    assert not ev.allclose([torch.ones(1)], [torch.ones(1), torch.ones(1)])  # length mismatch
    assert ev.allclose(1, 1) and not ev.allclose(1, 2)


def test_integer_outputs_are_compared_exactly():
    a = torch.tensor([1000, 2000])
    assert ev.allclose(a, a.clone())
    assert not ev.allclose(a, torch.tensor([1001, 2000]))  # inside atol/rtol, still wrong
    x = torch.tensor([1.0, float("nan")])
    assert ev.allclose(x, x.clone(), exact=True)
    assert not ev.allclose(torch.tensor([1.0]), torch.tensor([1.0 + 1e-6]), exact=True)
    assert ev.bit_equal(torch.tensor([0.0]), torch.tensor([0.0])) and not ev.bit_equal(torch.tensor([0.0]), torch.tensor([-0.0]))
    quiet = torch.tensor([0x7FC0, 0x3F80], dtype=torch.int16).view(torch.bfloat16)
    other = torch.tensor([-1, 0x3F80], dtype=torch.int16).view(torch.bfloat16)      # another NaN payload
    assert ev.bit_equal(quiet, other) and not ev.bit_equal(quiet, other.flip(0))


def test_cpu_bench_call_count():
    calls = []
    ev.cpu_bench(lambda: calls.append(1), num_runs=7)
    assert len(calls) == 10 + 7


def _fast_p(is_correct, baseline, actual, n, p):
    keep = [i for i in range(n) if is_correct[i]]
    sp = np.array([baseline[i] for i in keep]) / np.array([actual[i] for i in keep]) if keep else np.array([])
    return float(np.sum(sp > p)) / n if n else 0.0


@pytest.mark.parametrize("n", [5, 10, 50, 100])
@pytest.mark.parametrize("p", [0, 1, 1.5, 2])
def test_perf_at_p_equals_fast_p(n, p):
    rng = np.random.default_rng(n * 10 + int(p * 2))
    correct = rng.integers(0, 2, n)
    perf = rng.uniform(0.5, 2, n)
    actual = rng.integers(1, 101, n).astype(float)
    expected = _fast_p(correct, actual * perf, actual, n, p)
    assert float(ev.perf_at_p(correct.tolist(), perf.tolist(), p)) == pytest.approx(expected, abs=1e-6)


def test_perf_at_p_length_check():
    with pytest.raises(AssertionError):
        ev.perf_at_p([1, 0], [1.0], 1.0)


def test_eval_correctness_counts_and_errors():
    op = torch.ops.aten.relu.default
    tests = [Case(lambda: torch.randn(8)), Case(lambda: torch.randn(3, 3))]
    score, results = ev.eval_correctness(op, op, tests)
    assert score == 1.0 and len(results) == 2 and all(r.is_correct and r.op_name == "relu.default" for r in results)
    score, results = ev.eval_correctness(op, lambda x: torch.full_like(x, 42.0), tests)
    assert score == 0.0 and results[0].max_abs_error > 1

    def boom(x):
        raise RuntimeError("kaput")

    score, results = ev.eval_correctness(op, boom, tests)
    assert score == 0.0 and "kaput" in results[0].error_msg and "RuntimeError" in results[0].error_type
    assert ev.eval_correctness(op, op, []) == (0.0, [])


def test_eval_performance_failed_impl_counts_as_one():
    op = torch.ops.aten.relu.default
    tests = [Case(lambda: torch.randn(64))]
    score, results = ev.eval_performance(op, lambda x: torch.full_like(x, 42.0), tests)
    assert float(score) == pytest.approx(1.0) and not results[0].successfully_ran and results[0].speedup is None
    score, results = ev.eval_performance(op, op, tests)
    assert results[0].successfully_ran and results[0].speedup > 0


def _streamy(x):
    s = torch.cuda.Stream()
    return x, s


def test_eval_one_op_skips_stream_creators():
    op = torch.ops.aten.relu.default
    c, p, cr, pr = ev.eval_one_op(op, _streamy, [Case(lambda: torch.randn(2))], [Case(lambda: torch.randn(2))])
    assert c == 0 and p == 1.0 and cr[0].error_msg == "Skipped: uses CUDA stream" and pr[0].speedup == 0


def test_smoke_suite_with_aten_backend():
    backend = AtenBackend()
    corr, perf = [], []
    for t in SmokeTestSuite:
        assert t.op in backend
        c, p, cr, pr = ev.eval_one_op(t.op, backend[t.op], t.correctness_tests, t.performance_tests)
        assert c > 0 and p > 0.1 and len(cr) == 1 and len(pr) == 1
        corr.append(c)
        perf.append(float(p))
    assert np.mean(corr) >= 0.8 and np.exp(np.mean(np.log(perf))) >= 0.5
