"""Command line of the evaluation harness.

    python -m backendbench_amd.scripts.main --suite smoke --backend directory --ops-directory generated_kernels

Same flow and flags as BackendBench/scripts/main.py:43-325 for the parts this build
carries: pick a suite and a backend, evaluate every op the backend implements, print the
three scores, write the result files (default log dir of the directory backend = its ops
directory).  Suites: `smoke` (the reference's), `baseline` (this operator set's own cases)
and `trace` (argument strings from a file, the reference's TorchBench text format).
"""

import datetime
import logging
import os
import sys

import click
import torch

from .. import backends, eval as evaluator
from ..output import save_results
from ..suite import BaselineTestSuite, SmokeTestSuite

logger = logging.getLogger(__name__)


def setup_logging(level):
    logging.basicConfig(level=getattr(logging, str(level).upper(), logging.INFO),
                        format="[%(asctime)s][%(levelname)s][%(filename)s] %(message)s", datefmt="%Y-%m-%d %H:%M:%S")


@click.command()
@click.option("--log-level", default=os.getenv("LOG_LEVEL", "INFO"),
              type=click.Choice(["DEBUG", "INFO", "WARNING", "ERROR", "CRITICAL"], case_sensitive=False))
@click.option("--suite", default="smoke", type=click.Choice(["smoke", "baseline", "trace"]), help="Which suite to run")
@click.option("--backend", default="aten", type=click.Choice(["aten", "directory"]), help="Which backend to run")
@click.option("--ops", default=None, type=str, help="Comma-separated list of ops to run")
@click.option("--topn-inputs", "--topn", default=None, type=int, help="Largest N inputs per op (trace suite only)")
@click.option("--trace-path", default=None, type=str, help="File of argument strings for the trace suite")
@click.option("--ops-directory", default="generated_kernels", type=str, help="Directory of operator folders")
@click.option("--log-dir", default=None, type=str,
              help="Output directory (default: the ops directory for the directory backend, else a timestamped one)")
@click.option("--disable-output-logs", default=False, is_flag=True, help="Do not write result files")
@click.option("--p", default=1.0, type=float, help="Speed-up threshold of the perf@p score")
@click.option("--device", default=None, type=str, help="Device of the baseline suite's tensors (default: cuda if present)")
@click.option("--scale", default=1.0, type=float, help="Shrink factor for the baseline suite's headline shapes")
def cli(log_level, suite, backend, ops, topn_inputs, trace_path, ops_directory, log_dir, disable_output_logs, p,
        device, scale):
    if suite != "trace" and topn_inputs is not None:
        raise ValueError("topn-inputs is only supported for the trace suite")
    setup_logging(log_level)
    op_filter = ops.split(",") if ops else None
    device = device or ("cuda" if torch.cuda.is_available() else "cpu")
    if suite == "smoke":
        tests = SmokeTestSuite
    elif suite == "baseline":
        tests = BaselineTestSuite(device, scale, op_filter)
    else:
        from ..suite.trace import TraceTestSuite

        if not trace_path:
            raise ValueError("--trace-path is required for the trace suite")
        tests = TraceTestSuite("trace", trace_path, filter=op_filter, topn=topn_inputs)

    backend_name = backend
    backend = backends.DirectoryBackend(ops_directory) if backend == "directory" else backends.AtenBackend()
    if not log_dir:
        log_dir = ops_directory if backend_name == "directory" else \
            f"backendbench_output_{datetime.datetime.now().strftime('%Y%m%d_%H%M%S')}"

    overall_correct, overall_perf, c_all, p_all = [], [], [], []
    for test in tests:
        if test.op not in backend:
            continue
        logger.debug(test.op)
        _, perf, c_res, p_res = evaluator.eval_one_op(test.op, backend[test.op], test.correctness_tests,
                                                      test.performance_tests)
        overall_correct.append(all(r.is_correct for r in c_res))
        overall_perf.append(perf)
        c_all.extend(c_res)
        p_all.extend(p_res)
        if torch.cuda.is_available():
            logger.debug("max memory allocated: %s", f"{torch.cuda.max_memory_allocated():,}")

    mean_correctness = torch.tensor(overall_correct).float().mean().item()
    geomean_perf = torch.tensor([float(x) for x in overall_perf]).log().mean().exp().item()
    perf_at_p_score = evaluator.perf_at_p(overall_correct, [float(x) for x in overall_perf], p)
    print(f"correctness score (mean pass rate over all operators): {mean_correctness:.2f}")
    print(f"performance score (geomean speedup over all operators): {geomean_perf:.2f}")
    print(f"perf@p score (rate of correct samples with a speedup greater than p, p={p}): {perf_at_p_score:.2f}")
    command = "python -m backendbench_amd.scripts.main " + " ".join(sys.argv[1:])
    if not disable_output_logs:
        save_results(c_all, p_all, log_dir, command=command, mean_correctness=mean_correctness,
                     geomean_perf=geomean_perf, perf_at_p_score=perf_at_p_score, p=p)


if __name__ == "__main__":
    cli()
