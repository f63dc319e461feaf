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

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, GB/s
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, TFLOP/s
# HBM bytes per launch from hardware counters (FETCH_SIZE + WRITE_SIZE, each scaled by what the
# same counter reads for a plain 128 MiB copy); measured once per kernel with rocprofv3 --pmc,
# summary in profiles/C2_row_kernels__softmax_layer_norm.md.  Not re-measured by this script.
MEASURED_TRAFFIC_BYTES = {"C2.layer_norm": 138_790_000, "C2.softmax": 134_300_000}


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
    ap.add_argument("--only-op", default=None, help="time just this per-op row (for profilers); 'calib.copy' = plain copy, 'calib.mm' = a product of --shape in --dtype")
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
    from backendbench_amd.suite import perf_cases

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    backend = DirectoryBackend(os.path.join(ROOT, "generated_kernels"))
    cases = perf_cases(args.scale)
    by_key = {c.key: c for c in cases}

    def impl_of(case):
        return backend[case.op]

    # ------------------------------------------------------------ profiler mode
    # One op only, timed exactly like its per_op row, so that a profiler's per-kernel average
    # covers the same launches.  "calib.copy" is a plain 128 MiB -> 128 MiB copy with the
    # library's copy kernel (known traffic, for scaling hardware byte counters).
    if args.only_op == "calib.mfma":
        print(json.dumps(calib_mfma_f64(dev, args.variant or 16) if args.dtype == "f64" else calib_mfma(dev, args.fill, args.variant)))
        return
    if args.only_op == "calib.mm":
        M, K, N = (int(v) for v in args.shape.split(","))
        dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32, "f64": torch.float64}[args.dtype]
        a = torch.randn(M, K, device=dev).to(dt)
        b = (torch.randn(K, N, device=dev) * 0.02).to(dt)
        ms, how = graph_bench(backend[torch.ops.aten.mm.default], [a, b], {})
        tiles = -(-M // 256) * -(-N // 256)
        print(json.dumps({"only_op": "calib.mm", "shape": [M, K, N], "dtype": args.dtype, "ms": round(ms, 5),
                          "tflops": round(2.0 * M * K * N / (ms * 1e-3) / 1e12, 1), "tiles_256x256": tiles,
                          "rounds_of_256_cus": round(tiles / 256, 3), "timing": how}))
        return
    if args.only_op and args.trace:
        print(json.dumps(gemm_trace(by_key[args.only_op], dev, args.fill)))
        return
    if args.only_op and args.ablate is not None:
        print(json.dumps(gemm_ablate(by_key[args.only_op], dev, args.ablate, args.fill)))
        return
    if args.only_op:
        if args.only_op == "calib.copy":
            from backendbench_amd.ops._common import copy_into

            src = torch.empty(32 * 2**20, dtype=torch.float32, device=dev).normal_()
            f, a, kw, work = (lambda s: copy_into(torch.empty_like(s), s)), [src], {}, 2 * src.numel() * 4
        else:
            case = by_key[args.only_op]
            a, kw = case.make(dev)
            f, work = impl_of(case), case.work
            if args.fill:
                for t in a:
                    if isinstance(t, torch.Tensor) and t.dtype.is_floating_point:
                        if args.fill == "sign":
                            t.copy_(torch.randint(-1, 2, t.shape, device=t.device).to(t.dtype))
                        else:
                            t.fill_(0.0 if args.fill == "zeros" else 1.0)
        ms, how = graph_bench(f, a, kw)
        print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "work": work, "timing": how,
                          **({"fill": args.fill} if args.fill else {})}))
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

    rows = {r["op"]: r for r in per_op}
    # dominant kernel of the step = the op with the largest share of a step's GPU time
    roofline = None
    timed = [rows[k] for k in step_keys if k in rows]
    if timed:
        dom = max(timed, key=lambda r: r["ms"])
        roofline = {"bound": "hbm", "kernel": dom["op"], "achieved": dom["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(dom["gbs"] / HBM_PEAK_GBS, 4),
                    "traffic": MEASURED_TRAFFIC_BYTES.get(dom["op"]) if args.scale == 1.0 else None,
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
        "roofline": roofline, "cpu_baseline": cpu_baseline,
        "geomean_speedup_vs_cpu": geomean, "per_op": per_op,
    }
    print(json.dumps(line))


def copy_ms_for(nbytes, dev, cache):
    """Mean ms per launch of the library's flat copy kernel moving `nbytes` in total (half read,
    half written), with graph_bench's recipe: the size-matched ceiling of a memory-bound row
    (launch ramp and tail included, which dominate rows of a few tens of megabytes)."""
    import torch

    from backendbench_amd.ops._common import copy_into

    n = max(1024, (nbytes // 2) // 4096 * 1024)  # fp32 elements of the source
    if n not in cache:
        src = torch.empty(n, dtype=torch.float32, device=dev).normal_()
        cache[n] = graph_bench(lambda s: copy_into(torch.empty_like(s), s), [src], {})[0]
        del src
    return cache[n]


def calib_mfma(dev, fill=None, variant=0, blocks=256, steps=2752, launches=20):
    """Sustained rate of the mm kernel's MFMA stream with no memory traffic (mi355_calib_mfma): one
    workgroup of four waves per CU, each wave a 128 x 128 register tile, `steps` 32-k steps per
    launch (eight times the K loop of the [4096,11008] x [11008,4096] product).  Operand data as
    the GEMM configuration prescribes (left N(0,1), right N(0,0.02), bf16) unless `fill` overrides
    it: what this loop sustains is the ceiling the power / clock envelope leaves a GEMM on that data."""
    import torch

    from backendbench_amd import _lib

    lib = _lib.load()
    g = torch.Generator().manual_seed(0)
    n = blocks * 256 * 16 * 8  # bf16 elements per operand buffer
    a = torch.randn(n, generator=g).bfloat16()
    b = (torch.randn(n, generator=g) * 0.02).bfloat16()
    if fill == "zeros":
        a.zero_(), b.zero_()
    elif fill == "ones":
        a.fill_(1.0), b.fill_(1.0)
    elif fill == "sign":
        a = torch.randint(-1, 2, (n,), generator=g).bfloat16()
        b = torch.randint(-1, 2, (n,), generator=g).bfloat16()
    a, b = a.to(dev), b.to(dev)
    out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    stream = _lib.current_stream_handle()

    def run():
        _lib.check(lib.mi355_calib_mfma(a.data_ptr(), b.data_ptr(), out.data_ptr(), _lib.BF16, blocks, steps, variant, stream))

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / launches
    flops = blocks * 4 * steps * 2 * 128 * 128 * 32
    tf = flops / (ms * 1e-3) / 1e12
    return {"only_op": "calib.mfma", "variant": variant, "fill": fill or "N(0,1) x N(0,0.02)", "ms": round(ms, 4),
            "flops": flops, "tflops": round(tf, 1), "frac_of_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
            "timing": f"{launches} launches of {blocks} x 4 waves x {steps} steps, events around the loop"}


def calib_mfma_f64(dev, waves, blocks=256, steps=20000, launches=5):
    """Issue rate of v_mfma_f64_16x16x4_f64 with `waves` waves per workgroup, one workgroup per CU, eight
    independent accumulator blocks per wave, no memory traffic (mi355_calib_mfma with dtype f64)."""
    import torch

    from backendbench_amd import _lib

    lib = _lib.load()
    g = torch.Generator().manual_seed(0)
    a = torch.randn(256, generator=g, dtype=torch.float64).to(dev)
    b = torch.randn(256, generator=g, dtype=torch.float64).to(dev)
    out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    stream = _lib.current_stream_handle()

    def run():
        _lib.check(lib.mi355_calib_mfma(a.data_ptr(), b.data_ptr(), out.data_ptr(), _lib.F64, blocks, steps, waves, stream))

    run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / launches
    flops = blocks * waves * steps * 8 * 2048
    tf = flops / (ms * 1e-3) / 1e12
    return {"only_op": "calib.mfma", "dtype": "f64", "waves_per_workgroup": waves, "ms": round(ms, 4), "flops": flops,
            "tflops": round(tf, 1), "frac_of_peak": round(tf / 78.6, 4),
            "ns_per_mfma_and_wave": round(ms * 1e6 / (steps * 8), 1),
            "timing": f"{launches} launches of {blocks} x {waves} waves x {steps} rounds of 8 MFMAs, events around the loop"}


def gemm_ablate(case, dev, bits, fill=None, launches=40):
    """The row's mm through the ablation build `bits` (see csrc/gemm_x16.hip): events around `launches`
    back-to-back launches after a warm-up.  Timing only - the build leaves work out, its results are wrong.
    MI355_GEMM_TILE in the environment applies as usual (x16 = one workgroup per tile)."""
    import ctypes

    import torch

    from backendbench_amd import _build, _lib

    path = _build.ablate_lib_path(bits)
    if not path.exists():
        raise RuntimeError(f"{path} is missing: python -m backendbench_amd._build --ablate {bits}")
    lib = ctypes.CDLL(str(path))
    fn = lib.mi355_gemm
    fn.restype, fn.argtypes = _lib.SIGNATURES["mi355_gemm"]
    (a, b), _ = case.make(dev)
    if fill:
        for t in (a, b):
            t.copy_(torch.randint(-1, 2, t.shape, device=dev).to(t.dtype)) if fill == "sign" else t.fill_(0.0 if fill == "zeros" else 1.0)
    M, K = a.shape
    N = b.shape[1]
    out = torch.empty(M, N, dtype=a.dtype, device=dev)

    def run():
        _lib.check(fn(a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), None, 0, 0,
                      out.data_ptr(), M, N, K, 1.0, 0.0, _lib.dtype_code(a.dtype), None, 0, _lib.current_stream_handle()))

    for _ in range(3 * launches):  # the first dozens of launches of a process run slower (clocks, power state)
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / launches
    flops = 2.0 * M * N * K
    return {"only_op": case.key, "ablate": bits, "fill": fill or "as configured", "ms": round(ms, 5),
            "tflops_nominal": round(flops / (ms * 1e-3) / 1e12, 1),
            "timing": f"events around {launches} back-to-back launches; results are wrong by construction"}


def gemm_trace(case, dev, fill=None):
    """One mm of this row through the stamped diagnostic build (see the MI355_GEMM_TRACE blocks in
    csrc/gemm_x16.hip and csrc/gemm.hip for the record layout): mean shader-clock ticks per phase of a
    tile and per pair of steps of the K loop (a step = 32 k: a half-stage of the 16x16x32 kernel, 64
    MFMAs of 16 clocks, or a step of the 32x32x16 kernels, 32 MFMAs of 32 clocks), the gap between two
    tiles on one CU, and ticks per microsecond of kernel time (the average shader clock, which is
    what moves with the operand data).  MI355_GEMM_WAVES=4 in the environment selects the
    32x32x16 four-wave kernel instead of the 16x16x32 one."""
    import ctypes

    import numpy as np
    import torch

    from backendbench_amd import _build, _lib

    if not _build.TRACE_LIB_PATH.exists():
        raise RuntimeError(f"{_build.TRACE_LIB_PATH} is missing: python -m backendbench_amd._build --trace")
    lib = ctypes.CDLL(str(_build.TRACE_LIB_PATH))
    fn = lib.mi355_gemm
    fn.restype, fn.argtypes = _lib.SIGNATURES["mi355_gemm"]
    (a, b), _ = case.make(dev)
    if fill:
        for t in (a, b):
            t.copy_(torch.randint(-1, 2, t.shape, device=dev).to(t.dtype)) if fill == "sign" else t.fill_(0.0 if fill == "zeros" else 1.0)
    M, K = a.shape
    N = b.shape[1]
    out = torch.empty(M, N, dtype=a.dtype, device=dev)
    ws = torch.zeros(1 << 20, dtype=torch.int64, device=dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        ws.zero_()
        e0.record()
        _lib.check(fn(a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), None, 0, 0,
                      out.data_ptr(), M, N, K, 1.0, 0.0, _lib.dtype_code(a.dtype), ws.data_ptr(), ws.numel() * 8,
                      _lib.current_stream_handle()))
        e1.record()
        torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3
    rec = ws.cpu().numpy().reshape(-1, 4, 16)
    rec = rec[rec[:, 0, 7] > 0]
    w0 = rec[:, 0, :].astype(np.float64)
    iters = w0[:, 7]
    entry, begin, end, drained, stored = w0[:, 12], w0[:, 10], w0[:, 13], w0[:, 14], w0[:, 15]
    hw = rec[:, 0, 11]
    cu_key = (np.arange(len(rec)) % 8) * 4096 + (hw & 0xFF00)  # XCD (block % 8), SE / SH / CU bits of HW_ID
    gaps = []
    for k in np.unique(cu_key):
        idx = np.where(cu_key == k)[0]
        idx = idx[np.argsort(entry[idx])]
        gaps += list(entry[idx[1:]] - stored[idx[:-1]])
    per_step = (w0[:, :6] / iters[:, None]).mean(axis=0)
    names = ["even_issue", "even_fill_wait", "even_barrier", "odd_issue", "odd_fill_wait", "odd_barrier_and_back_edge"]
    whole = float(np.mean(stored - entry))
    return {"only_op": case.key, "trace": True, "fill": fill or "as configured", "kernel_us": round(us, 1), "tiles": int(len(rec)),
            "ticks_per_step_pair": {n: round(float(v), 1) for n, v in zip(names, per_step)},
            "mfma_ticks_per_step_pair_at_full_rate": 2048,
            "ticks_per_tile": {"prologue": round(float(np.mean(begin - entry))), "steady_loop": round(float(np.mean(end - begin))),
                               "remainder_and_drain": round(float(np.mean(drained - end))),
                               "epilogue_until_stored": round(float(np.mean(stored - drained))), "whole_tile": round(whole)},
            "ticks_between_tiles_on_a_cu": round(float(np.median(gaps))) if gaps and len(rec) > 256 else None,
            "rounds_of_tiles": round(len(rec) / 256, 3),
            "approx_ticks_per_us": round(whole * max(1.0, np.ceil(len(rec) / 256)) / us) if us > 0 else None}


def graph_bench(fn, args, kwargs, pool_bytes=768 * 2**20, target_ms=60.0):
    """Mean ms per launch of `fn`: a HIP graph holds one launch per member of a pool of
    argument copies (pool larger than the last-level cache, so no launch finds its inputs
    cached); the graph is replayed back to back and the whole run is bracketed by one pair of
    events on the launch stream.  Per-launch time = elapsed / launches: kernel time plus the
    graph's inter-kernel gap, without per-launch event or Python overhead."""
    import torch

    nbytes = sum(a.numel() * a.element_size() for a in args if isinstance(a, torch.Tensor))
    # at least four copies while they fit 6 GiB (inputs of a gigabyte: the gathers), else two (the 4.2 GB argmax)
    copies = max(4 if 4 * nbytes <= 6 * 2**30 else 2, min(24, math.ceil(pool_bytes / max(nbytes, 1))))
    # A replay costs about 2.3 us on top of its kernels (two launches per graph: + 1.2 us each, twelve: + 0.2):
    # a graph of few copies walks its pool more than once, so that every row carries about the same share.
    rounds = math.ceil(6 / copies)
    launches = copies * rounds
    clone = lambda seq: [x.clone() if isinstance(x, torch.Tensor) else x for x in seq]
    pool = [list(args)] + [clone(args) for _ in range(copies - 1)]
    for p in pool[:2]:
        fn(*p, **kwargs)
    torch.cuda.synchronize()
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            held = [fn(*p, **kwargs) for _ in range(rounds) for p in pool]
        run, per_run, how = graph.replay, launches, f"hip graph of {launches} launches over {copies} input copies, events around replays"
    except Exception as exc:  # noqa: BLE001
        print(f"bench.py: graph capture failed for this op ({exc}); eager launches", file=sys.stderr)
        run, per_run, how = (lambda: [fn(*p, **kwargs) for p in pool]), copies, "eager launches over input copies, events around the loop"
    run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    run()
    e1.record()
    torch.cuda.synchronize()
    once = max(e0.elapsed_time(e1), 1e-3)
    reps = max(3, min(2000, int(target_ms / once)))
    e0.record()
    for _ in range(reps):
        run()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (reps * per_run), how


def cpu_time_ms(case, args, kwargs, budget_s=2.0):
    """Mean ms per call of ATen on the host CPU for this row (the oracle), at full size, with the
    reference's CPU recipe (BackendBench/eval.py:149-159: 10 warm-up calls, then 100 timed calls
    with perf_counter, mean).  Rows that cost more than 10 ms per call (the GEMMs, the 4.2 GB
    argmax) keep the full-size call and run fewer repetitions, as many as fit `budget_s`; the
    counts are reported."""
    import torch

    from oracle import aten_cpu

    a = aten_cpu.to_cpu(list(args))
    kw = aten_cpu.to_cpu(dict(kwargs))
    t0 = time.perf_counter()
    case.op(*a, **kw)
    first = time.perf_counter() - t0
    if first < 0.010:
        warm, runs = 10, 100
    else:
        runs = max(3, min(100, int(budget_s / first)))
        warm = max(1, min(10, runs // 3))
    sec = aten_cpu.time_call(case.op, a, kw, warmup=warm, runs=runs)
    return round(sec * 1e3, 4), f"full size, {warm} warm-up + {runs} timed runs, {torch.get_num_threads()} threads"


if __name__ == "__main__":
    main()
