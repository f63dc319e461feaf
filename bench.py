#!/usr/bin/env python3
"""Benchmark of the directory backend's HIP kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A "step" is one pass of the headline row-op workload (the second of
the five benchmark configurations): `_softmax`, `native_layer_norm`, `sum` and `amax` over the last
dim of a bf16 [8192, 4096] tensor, each called once through the drop-in boundary
(DirectoryBackend -> `<folder>_kernel_impl` -> ctypes -> libmi355_aten.so).  Inputs are
resident in HBM before the clock starts; consecutive steps walk a pool of input copies larger
than the last-level cache, so every step reads from HBM.  `value` is the algorithmic bytes of
a step divided by the time of a step.

Beside the step loop the script times every headline row of all five configurations: `ms` is
the mean time per launch of a HIP graph that holds one launch per member of a pool of input
copies (cold inputs, one event pair around the replays; agrees with rocprofv3's per-kernel
average), `ms_flush_events` is the reference's own GPU recipe (flush the cache, one event pair
per repetition, mean).  It reports GB/s or TFLOP/s and the fraction of the MI355X peak per op
under "per_op", times ATen on the host CPU for the same calls ("cpu_baseline", bounded samples)
and reports the geometric mean speed-up over it.
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# HBM bytes per launch from hardware counters (FETCH_SIZE + WRITE_SIZE, each scaled by what the
# same counter reads for a plain 128 MiB copy): rocprofv3 --pmc runs of `bench.py --only-op <row>`,
# commands and tables in profiles/C2_row_kernels__softmax_layer_norm.md.  A profiler cannot run inside
# this script, so the figures are carried here and named as such in the output ("traffic_source").
MEASURED_TRAFFIC_BYTES = {"C2.layer_norm": 134_670_000, "C2.softmax": 134_280_000}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--launch", choices=["graph", "eager"], default="graph",
                    help="replay the step loop from a HIP graph (default) or launch eagerly from Python")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink factor for every shape (debug only)")
    ap.add_argument("--ops", default="all", help="comma-separated substrings of per-op rows to time, or 'none'")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-calib", action="store_true", help="skip the calibration block (plain copies, MFMA streams)")
    ap.add_argument("--only-op", default=None, help="time just this per-op row (for profilers); 'calib.copy' = plain copy, 'calib.mm' = a product of --shape in --dtype, "
                                                       "'calib.all' = the calibration block, 'e2e.gpt2' = a GPT-2-small forward with and without the override")
    ap.add_argument("--variant", type=int, default=0,
                    help="with --only-op calib.mfma: 0 = the 32x32x16 mm kernels' MFMA order, 1 = operands swapped between the "
                         "ports, 2 = the other operand held across MFMAs, 3 = v_mfma_f32_16x16x32, 4-9 = chained "
                         "accumulator updates, 10 = the 16x16x32 mm kernel's stream, 11-14 = its reorderings "
                         "(see mi355_calib_mfma in include/mi355_aten.h)")
    ap.add_argument("--ablate", type=int, default=None,
                    help="with --only-op C3.mm_up|C3.mm_down: time the GEMM through the measurement build that leaves "
                         "parts of the 16x16x32 kernel out (python -m backendbench_amd._build --ablate N; bits: 1 fills, "
                         "2 barriers, 4 LDS fragment reads, 8 fill waits, 16 epilogue stores, 32 epilogue); wrong results")
    ap.add_argument("--trace", action="store_true",
                    help="with --only-op C3.mm_up|C3.mm_down: run the cycle-stamped diagnostic build of the GEMM "
                         "(libmi355_gemm_trace.so) and print where a tile's shader-clock ticks go")
    ap.add_argument("--shape", default=None,
                    help="with --only-op calib.mm: M,K,N of a product [M,K] x [K,N] (--dtype, default bf16) timed like a C3 row, operands "
                         "drawn like C3's (how the time of a K = 4096 product moves with the number of 256x256 tiles)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32", "f64"],
                    help="with --only-op calib.mm: the operands' dtype; with --only-op calib.mfma: f64 times the fp64 MFMA "
                         "(--variant = waves per workgroup: 1, 4, 8, 16)")
    ap.add_argument("--fill", default=None, choices=["zeros", "ones", "sign"],
                    help="with --only-op: overwrite the floating-point inputs with zeros, ones or values from "
                         "{-1, 0, 1} (shows how far a kernel's time depends on the data through the power/clock envelope)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (every kernel works on one GPU's share); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels only run on an MI355X", file=sys.stderr)
        sys.exit(1)

    from backendbench_amd import eval as ev
    from backendbench_amd.backends import DirectoryBackend
    from backendbench_amd.suite import out_perf_cases, perf_cases

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    backend = DirectoryBackend(os.path.join(ROOT, "generated_kernels"))
    cases = perf_cases(args.scale)
    by_key = {c.key: c for c in cases}

    def impl_of(case):
        return backend[case.op]

    from backendbench_amd import measure
    from backendbench_amd.measure import HBM_PEAK_GBS, MFMA_BF16_PEAK_TFLOPS, copy_ms_for, cpu_time_ms, graph_bench

    # One op only (profilers, calibrations, diagnostics): backendbench_amd/measure.py
    if args.only_op:
        measure.only_op(args, backend, by_key, dev)
        return

    # ------------------------------------------------------------ headline step loop (C2)
    step_keys = ["C2.softmax", "C2.layer_norm", "C2.sum", "C2.amax"]
    step_cases = [by_key[k] for k in step_keys]
    step_bytes = sum(c.work for c in step_cases)
    (x0, _, _), _ = by_key["C2.softmax"].make(dev)
    (_, nshape, gamma, beta, eps), _ = by_key["C2.layer_norm"].make(dev)
    pool_n = max(8, math.ceil(1.5 * 2**30 / (x0.numel() * x0.element_size())) // 4 * 4)  # >= 1.5 GiB of inputs, multiple of 4
    pool = [x0] + [x0.clone() for _ in range(pool_n - 1)]
    softmax, layer_norm = impl_of(by_key["C2.softmax"]), impl_of(by_key["C2.layer_norm"])
    rsum, ramax = impl_of(by_key["C2.sum"]), impl_of(by_key["C2.amax"])

    def step(i):
        # Each of the four calls takes its own member of the pool, and a member comes round again
        # only after pool_n - 1 other calls (1.5 GiB of traffic): no call finds its input in the
        # 256 MB last-level cache, the previous call's included.
        j = 4 * i
        return (softmax(pool[j % pool_n], -1, False), layer_norm(pool[(j + 1) % pool_n], nshape, gamma, beta, eps),
                rsum(pool[(j + 2) % pool_n], [-1]), ramax(pool[(j + 3) % pool_n], [-1]))

    for i in range(3):  # first calls: library load, attribute set-up, allocator warm-up
        keep = step(i)
    torch.cuda.synchronize()

    # One step's outputs against the oracle before anything is timed.
    from oracle import aten_cpu

    verified = True
    calls = [(by_key["C2.softmax"], [x0, -1, False]), (by_key["C2.layer_norm"], [x0, nshape, gamma, beta, eps]),
             (by_key["C2.sum"], [x0, [-1]]), (by_key["C2.amax"], [x0, [-1]])]
    for case_k, a_k in calls:
        got = impl_of(case_k)(*a_k)
        torch.cuda.synchronize()
        if not ev.allclose(aten_cpu.reference(case_k.op, a_k, {}), aten_cpu.to_cpu(got)):
            verified = False
            print(f"bench.py: {case_k.key} differs from the oracle", file=sys.stderr)
    if not verified:
        sys.exit(3)

    launch_mode = args.launch
    per_graph = pool_n // 4  # steps in one walk over the pool
    graphs = {}

    def graph_of(n_steps):
        """HIP graph of `n_steps` consecutive steps (captured once per length)."""
        if n_steps not in graphs:
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                held = [step(i) for i in range(n_steps)]
            graphs[n_steps] = (gr, held)
        return graphs[n_steps][0]

    if launch_mode == "graph":
        try:
            graph_of(per_graph)
            for n in {args.steps % per_graph, args.warmup % per_graph} - {0}:
                graph_of(n)
            torch.cuda.synchronize()
        except Exception as exc:  # noqa: BLE001
            print(f"bench.py: graph capture failed ({exc}); falling back to eager launches", file=sys.stderr)
            graphs.clear()
            launch_mode = "eager"

    def run_steps(n):
        """Exactly n steps: whole walks over the pool, then one shorter graph for the remainder."""
        if launch_mode == "eager":
            for i in range(n):
                step(i)
            return
        for _ in range(n // per_graph):
            graphs[per_graph][0].replay()
        if n % per_graph:
            graphs[n % per_graph][0].replay()

    K, W = args.steps, args.warmup
    run_steps(W)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    run_steps(K)
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / K
    ms_per_step_events = ev0.elapsed_time(ev1) / K
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    graphs.clear()
    keep = None

    # ------------------------------------------------------------ per-op timings
    want = None if args.ops == "all" else ([] if args.ops == "none" else args.ops.split(","))
    per_op = []
    cpu_times = {}
    copy_cache = {}
    for case in cases:
        if want is not None and not any(w in case.key for w in want):
            continue
        a, kw = case.make(dev)
        f = impl_of(case)
        ms, how = graph_bench(f, a, kw)
        row = {"op": case.key, "ms": round(ms, 5), "timing": how,
               "ms_flush_events": round(ev.gpu_bench(lambda: f(*a, **kw)), 5)}
        if case.bound == "hbm":
            gbs = case.work / (ms * 1e-3) / 1e9
            row.update(bound="hbm", bytes=int(case.work), gbs=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 4))
            # what a plain copy of the same number of bytes (half read, half written) reaches, timed the same way
            copy_ms = copy_ms_for(int(case.work), dev, copy_cache)
            row.update(copy_ms_same_bytes=round(copy_ms, 5), vs_copy=round(copy_ms / ms, 3))
        else:
            tf = case.work / (ms * 1e-3) / 1e12
            row.update(bound="mfma", flops=int(case.work), tflops=round(tf, 1), frac=round(tf / MFMA_BF16_PEAK_TFLOPS, 4))
        if not args.no_cpu:
            row["cpu_ms"], row["cpu_sample"] = cpu_time_ms(case, a, kw)
            row["speedup_vs_cpu"] = round(row["cpu_ms"] / ms, 1)
            cpu_times[case.key] = row["cpu_ms"]
        per_op.append(row)
        del a, kw
        torch.cuda.empty_cache()

    # out= overloads at four headline shapes: `out` has the result's shape and dtype, so the kernels write into
    # it directly and the row should cost what the functional row does (vs_functional = functional ms / this ms).
    by_ms = {r["op"]: r["ms"] for r in per_op}
    out_rows = []
    wanted_out = {"O.add_out": "C1.add", "O.relu_out": "C1.relu", "O.softmax_out": "C2.softmax", "O.mm_up_out": "C3.mm_up"}
    for case in out_perf_cases(args.scale):
        base = wanted_out.get(case.key)
        if base is None or base not in by_ms:
            continue
        a, kw = case.make(dev)
        ms, how = graph_bench(backend[case.op], a, kw)
        out_rows.append({"op": case.key, "ms": round(ms, 5), "functional_row": base, "vs_functional": round(by_ms[base] / ms, 3), "timing": how})
        del a, kw
        torch.cuda.empty_cache()

    # What the chip sustains in this very run: plain copies over five sizes and the GEMM kernels' MFMA
    # streams without memory traffic.  Every row is then also stated against that measured ceiling.
    calib = None
    if not args.no_calib and args.scale == 1.0:
        calib = measure.calib_block(dev)
        fit = calib["copy_fit"]
        stream = calib["mfma"]["x16_stream_gemm_data"]["tflops"]
        for r in per_op:
            if r["bound"] == "hbm":
                fit_ms = fit["intercept_us"] * 1e-3 + r["bytes"] / (fit["asymptote_gbs"] * 1e9) * 1e3
                r["copy_fit_ms"] = round(fit_ms, 5)          # a plain copy of this many bytes, from the fitted line
                r["vs_copy_fit"] = round(fit_ms / r["ms"], 3)
            else:
                r["frac_of_measured_stream"] = round(r["tflops"] / stream, 4)  # of the 16x16x32 MFMA stream on this data
    rows = {r["op"]: r for r in per_op}
    # dominant kernel of the step = the op with the largest share of a step's GPU time
    roofline = None
    timed = [rows[k] for k in step_keys if k in rows]
    if timed:
        dom = max(timed, key=lambda r: r["ms"])
        roofline = {"bound": "hbm", "kernel": dom["op"], "achieved": dom["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(dom["gbs"] / HBM_PEAK_GBS, 4),
                    "traffic": MEASURED_TRAFFIC_BYTES.get(dom["op"]) if args.scale == 1.0 else None,
                    "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --only-op " + dom["op"] + "`, scaled by a 128 MiB copy's (profiles/)",
                    "bytes_per_launch": dom["bytes"], "avg_launch_ms": dom["ms"],
                    "timing": dom["timing"]}
    cpu_baseline = None
    if not args.no_cpu and all(k in cpu_times for k in step_keys):
        cpu_ms = sum(cpu_times[k] for k in step_keys)
        cpu_baseline = {"value": round(step_bytes / (cpu_ms * 1e-3) / 1e9, 2), "unit": "GB/s",
                        "cores": torch.get_num_threads(), "kind": "port",
                        "sample": "ATen CPU kernels (the oracle) on the same four calls at full size, 10 warm-up + 100 "
                                  "timed runs each (the reference's CPU recipe; see per_op[].cpu_sample)",
                        "ms_per_step": round(cpu_ms, 3), "host_cpus": os.cpu_count()}
    geomean = None
    sp = [r["speedup_vs_cpu"] for r in per_op if "speedup_vs_cpu" in r]
    if sp:
        geomean = round(math.exp(sum(math.log(s) for s in sp) / len(sp)), 1)

    line = {
        "metric": "per-op GB/s or TFLOP/s + % of roofline on 1 MI355X; geomean speedup vs aten CPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 storage, fp32 accumulate", "data": "synthetic (seeded N(0,2) on CPU, copied to HBM)",
        "ms_per_step_events": round(ms_per_step_events, 5), "outputs_checked_against_oracle": verified,
        "config": {"workload": "C2 row ops on bf16 [8192,4096]: _softmax(dim=-1) + native_layer_norm([4096]) + "
                               "sum(dim=-1) + amax(dim=-1), one call each per step, each on its own copy of the input",
                   "bytes_per_step": int(step_bytes), "launch": launch_mode, "input_pool": pool_n,
                   "scale": args.scale},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "calib": calib,
        "geomean_speedup_vs_cpu": geomean, "per_op": per_op, "out_overloads": out_rows,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
