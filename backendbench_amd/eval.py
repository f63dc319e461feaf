"""Evaluator: correctness against the ATen reference and speed-up over it.

Host-side mirror of BackendBench/eval.py (semantics, not code):
  * the reference result is `op(*args, **kwargs)` on the very same argument objects
    (eval.py:99-100);
  * results match when torch.testing.assert_close passes with atol = rtol = 1e-2 and
    equal_nan=True, recursing through lists/tuples (eval.py:68-90) — dtype, device and
    shape are part of that check, strides are not;
  * a performance test whose implementation fails or mismatches counts as speed-up 1.0
    (eval.py:181-220); the op score is the geometric mean of speed-ups (:222-224);
  * an implementation whose source creates streams is not run: correctness 0, perf 1.0
    (eval.py:236-262).
Stricter than the reference where the outputs are indices or copies: integer/bool outputs
and the results of EXACT_OPS must be bit-identical.
"""

import logging
import math
import time
import traceback
from dataclasses import dataclass
from typing import Optional, List, Tuple

import torch

from .utils import compute_errors, serialize_args, uses_cuda_stream

logger = logging.getLogger(__name__)

ATOL = 1e-2
RTOL = 1e-2
# Ops whose floating-point outputs are copies of input elements: compared bit for bit.
EXACT_OPS = {"index_select.default", "embedding.default", "gather.default", "argmax.default", "where.self"}


@dataclass
class CorrectnessTestResult:
    op_name: str
    args: str
    is_correct: bool = False
    error_msg: str = ""
    error_type: str = ""
    traceback: str = ""
    max_abs_error: float = -math.inf
    max_rel_error: float = -math.inf
    test_type: str = "correctness"


@dataclass
class PerformanceTestResult:
    op_name: str
    args: str
    speedup: float
    benchmark_time_ms: float
    reference_time_ms: float
    error_msg: str = ""
    successfully_ran: bool = False
    test_type: str = "performance"
    # Roofline columns (not in the reference's record, BackendBench/eval.py:36-46): filled when the
    # suite's test says how much algorithmic work one call is (the `baseline` suite's headline rows).
    algorithmic_work: Optional[float] = None   # bytes (bound "hbm") or flop (bound "mfma") per call
    bound: Optional[str] = None
    achieved: Optional[float] = None           # GB/s or TFLOP/s at benchmark_time_ms
    achieved_unit: Optional[str] = None
    roofline_frac: Optional[float] = None      # achieved / MI355X peak (8 TB/s HBM, 2.5 PFLOP/s dense bf16 MFMA)


_EXC_TEMPLATE = """
Exception raised for {op}:
    args: {args}
    exc: {exc}
    traceback: {tb}
"""


def format_exception(exc, op, args, kwargs, tb=None):
    name = getattr(op, "__name__", str(op))
    return _EXC_TEMPLATE.format(op=name, args=serialize_args(args, kwargs), exc=exc, tb=tb)


_INT_VIEW = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def bit_equal(a, b):
    """Same dtype, shape and bit pattern (so -0.0 != 0.0), except that any NaN equals any NaN:
    NaN payloads are not part of the contract (ATen's own CPU gather rewrites the payload of
    bf16 NaNs it copies)."""
    if not (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor)):
        return a == b
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    if a.numel() == 0:
        return True
    b = b.to(a.device)
    if a.dtype == torch.bool:
        return torch.equal(a, b)
    view = _INT_VIEW[a.element_size()]
    a, b = a.contiguous(), b.contiguous()
    ai, bi = a.view(view), b.view(view)
    if a.dtype.is_floating_point:
        nan_a, nan_b = a != a, b != b
        if not torch.equal(nan_a, nan_b):
            return False
        return torch.equal(ai[~nan_a], bi[~nan_a])
    return torch.equal(ai, bi)


def _walk_pairs(a, b):
    """Left-to-right leaves of two parallel nests (explicit stack: no recursion limit)."""
    stack = [(a, b)]
    while stack:
        x, y = stack.pop()
        if isinstance(x, (list, tuple)):
            assert isinstance(y, (list, tuple)) and len(x) == len(y)
            stack.extend(reversed(list(zip(x, y))))
        else:
            yield x, y


def allclose(a, b, atol=ATOL, rtol=RTOL, exact=False):
    """True when every leaf of `b` matches `a`: assert_close(atol, rtol, equal_nan) for
    tensors, == for anything else.  `exact` additionally demands identical bits; integer
    and bool tensors are always compared exactly."""
    try:
        for x, y in _walk_pairs(a, b):
            if isinstance(x, torch.Tensor):
                torch.testing.assert_close(x, y, equal_nan=True, atol=atol, rtol=rtol)
                if (exact or not (x.dtype.is_floating_point or x.dtype.is_complex)) and not bit_equal(x, y):
                    return False
            else:
                assert x == y
        return True
    except Exception:
        return False


def _is_exact_op(op):
    return getattr(op, "__name__", "") in EXACT_OPS


def _after_impl():
    # Indexing kernels report bad indices through a device flag; surface it per test.
    from .ops import check_index_errors

    check_index_errors()


def _own_outs(kwargs):
    """kwargs with every out= tensor (`out`, `out0`, ...) replaced by a clone.  The reference calls the operator
    and the implementation with the same kwargs (BackendBench/eval.py:99-102), so for an out= overload both
    would write into one tensor and the comparison would be of that tensor with itself."""
    return {k: (v.clone() if isinstance(v, torch.Tensor) and k.startswith("out") else v) for k, v in kwargs.items()}


def eval_correctness_test(op, impl, test) -> CorrectnessTestResult:
    args, kwargs = test.args, test.kwargs
    ref = op(*args, **_own_outs(kwargs))
    args_str = serialize_args(args, kwargs)
    try:
        res = impl(*args, **kwargs)
        _after_impl()
        ok = allclose(ref, res, exact=_is_exact_op(op))
        abs_err, rel_err = compute_errors(ref, res)
        return CorrectnessTestResult(op_name=op.__name__, args=args_str, is_correct=ok,
                                     max_abs_error=abs_err, max_rel_error=rel_err)
    except Exception as exc:
        tb = traceback.format_exc()
        msg = format_exception(exc, op, args, kwargs, tb)
        logger.warning(msg)
        return CorrectnessTestResult(op_name=op.__name__, args=args_str, is_correct=False, error_msg=msg,
                                     error_type=str(type(exc)), traceback=tb)


def eval_correctness(op, impl, tests) -> Tuple[float, List[CorrectnessTestResult]]:
    results = [eval_correctness_test(op, impl, t) for t in tests]
    if not results:
        logger.warning("No correctness tests available for %s", op)
        return 0.0, []
    return sum(r.is_correct for r in results) / len(results), results


def cpu_bench(fn, num_runs=100):
    """10 untimed calls, then the mean wall time of `num_runs` calls, in SECONDS."""
    for _ in range(10):
        fn()
    t0 = time.perf_counter()
    for _ in range(num_runs):
        fn()
    return (time.perf_counter() - t0) / num_runs


_flush_buf = {}


def _flush_cache(device):
    """Overwrite a buffer as large as the last-level cache so timed reads come from HBM."""
    buf = _flush_buf.get(device)
    if buf is None:
        buf = torch.empty(256 * 1024 * 1024, dtype=torch.int8, device=device)
        _flush_buf[device] = buf
    buf.zero_()


def gpu_bench(fn, warmup_ms=25.0, rep_ms=100.0):
    """Mean milliseconds per call measured with device events on the current stream.

    Same recipe as the timer the reference uses on GPUs (triton.testing.do_bench called
    with defaults at BackendBench/eval.py:179,195): one untimed call, a 5-call estimate,
    ~25 ms of warm-up, ~100 ms of timed repetitions, the cache flushed before every
    repetition, one event pair per repetition, mean of the repetitions.
    """
    device = torch.device("cuda", torch.cuda.current_device())
    fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        _flush_cache(device)
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate = start.elapsed_time(end) / 5
    n_warmup = max(1, int(warmup_ms / estimate))
    n_repeat = max(1, int(rep_ms / estimate))
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for _ in range(n_warmup):
        fn()
    for i in range(n_repeat):
        _flush_cache(device)
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return sum(times) / len(times)


def _bench_fn():
    return gpu_bench if torch.cuda.is_available() else cpu_bench


HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def roofline_columns(test, time_ms, on_gpu):
    """Roofline fields of a performance record from the work the suite's test declares
    (`test.case.work` / `.bound`); empty when it declares none or the time is not a GPU time."""
    case = getattr(test, "case", None)
    work, bound = getattr(case, "work", 0), getattr(case, "bound", None)
    if not on_gpu or not work or not time_ms or bound not in ("hbm", "mfma"):
        return {}
    if bound == "hbm":
        achieved, unit, peak = work / (time_ms * 1e-3) / 1e9, "GB/s", HBM_PEAK_GBS
    else:
        achieved, unit, peak = work / (time_ms * 1e-3) / 1e12, "TFLOP/s", MFMA_BF16_PEAK_TFLOPS
    return {"algorithmic_work": float(work), "bound": bound, "achieved": achieved, "achieved_unit": unit,
            "roofline_frac": achieved / peak}


def eval_performance(op, impl, tests) -> Tuple[float, List[PerformanceTestResult]]:
    bench = _bench_fn()
    base_times, test_times, results = [], [], []
    for test in tests:
        args, kwargs = test.args, test.kwargs  # drawn once: both sides time the same tensors
        args_str = serialize_args(args, kwargs)
        base = bench(lambda: op(*args, **kwargs))
        base_times.append(base)
        mine = base  # a failing implementation scores a speed-up of exactly 1.0
        try:
            ref = op(*args, **kwargs)
            res = impl(*args, **kwargs)
            _after_impl()
            if not allclose(ref, res, exact=_is_exact_op(op)):
                abs_err, rel_err = compute_errors(ref, res)
                raise ValueError(f"Reference and result tensors are not close: max absolute error {abs_err}, "
                                 f"max relative error {rel_err}")
            mine = bench(lambda: impl(*args, **kwargs))
            results.append(PerformanceTestResult(op_name=op.__name__, args=args_str, speedup=base / mine,
                                                 benchmark_time_ms=mine, reference_time_ms=base,
                                                 successfully_ran=True,
                                                 **roofline_columns(test, mine, bench is gpu_bench)))
        except Exception as exc:
            msg = format_exception(exc, op, args, kwargs, traceback.format_exc())
            results.append(PerformanceTestResult(op_name=op.__name__, args=args_str, speedup=None,
                                                 benchmark_time_ms=None, reference_time_ms=base, error_msg=msg,
                                                 successfully_ran=False))
        finally:
            test_times.append(mine)
    speedups = torch.tensor(base_times, dtype=torch.float64) / torch.tensor(test_times, dtype=torch.float64)
    return speedups.log().mean().exp().float(), results


def eval_one_op(op, impl, correctness_tests, performance_tests):
    """(correctness score, performance score, correctness results, performance results)."""
    if uses_cuda_stream(impl):
        logger.warning("Skipping %s because it uses CUDA stream", op.__name__)
        note = "Skipped: uses CUDA stream"
        c_res = [CorrectnessTestResult(op_name=op.__name__, args=serialize_args(t.args, t.kwargs),
                                       is_correct=False, error_msg=note) for t in correctness_tests]
        p_res = [PerformanceTestResult(op_name=op.__name__, args=serialize_args(t.args, t.kwargs), speedup=0,
                                       benchmark_time_ms=0, reference_time_ms=0, error_msg=note)
                 for t in performance_tests]
        return 0, 1.0, c_res, p_res
    c_score, c_res = eval_correctness(op, impl, correctness_tests)
    p_score, p_res = eval_performance(op, impl, performance_tests)
    return c_score, p_score, c_res, p_res


def perf_at_p(correctness, performance, p=1.0):
    """Fraction of ops that are correct AND faster than p x the reference (fast_p)."""
    assert len(correctness) == len(performance), "correctness and performance must have the same length"
    ok = torch.tensor(correctness).bool()
    fast = torch.tensor(performance) > p
    return torch.where(ok, fast, torch.zeros_like(fast)).float().mean()
