"""Measurement helpers behind bench.py: the timing recipes, the calibrations of what this chip sustains
(plain copies, the GEMM kernels' MFMA streams without memory traffic) and the profiler / diagnostic modes
`bench.py --only-op ...` dispatches to (one operator timed exactly like its per-op row, the cycle-stamped
and the ablation builds of the GEMM).  Nothing here is on the product path: the operator wrappers never
import this module.
"""

import collections
import json
import math
import os
import sys
import time

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, GB/s
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, TFLOP/s


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


def graph_bench(fn, args, kwargs, pool_bytes=768 * 2**20, target_ms=60.0, min_launches=24, keep=None):
    """Mean ms per launch of `fn`: a HIP graph holds one launch per member of a pool of
    argument copies (pool larger than the last-level cache, so no launch finds its inputs
    cached); the graph is replayed back to back and the whole run is bracketed by one pair of
    events on the launch stream.  Per-launch time = elapsed / launches: kernel time plus the
    graph's inter-kernel gap, without per-launch event or Python overhead."""
    import torch

    nbytes = sum(a.numel() * a.element_size() for a in args if isinstance(a, torch.Tensor))
    # at least four copies while they fit 6 GiB (inputs of a gigabyte: the gathers), else two (the 4.2 GB argmax)
    copies = max(4 if 4 * nbytes <= 6 * 2**30 else 2, min(24, math.ceil(pool_bytes / max(nbytes, 1))))
    # A replay costs about 2.3 us on top of its kernels (two launches per graph: + 1.2 us each, twelve: + 0.2,
    # twenty-four: + 0.1): a graph of fewer than 24 copies walks its pool more than once, so that every row
    # carries the same, small share of it (with six launches per graph the rows of 8 copies carried 0.3 us, those
    # of 24 copies 0.1 us, and the figure read 1 - 2 % above rocprofv3's per-kernel average for the former).
    rounds = math.ceil(min_launches / copies)
    launches = copies * rounds
    clone = lambda seq: [x.clone() if isinstance(x, torch.Tensor) else x for x in seq]
    pool = [list(args)] + [clone(args) for _ in range(copies - 1)]
    for p in pool[:2]:
        fn(*p, **kwargs)
    torch.cuda.synchronize()
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            # Results are dropped as a program's would be: the last `copies` stay alive (a result buffer comes round
            # again only after `copies` other launches, a pool's worth of traffic), the older ones return to the
            # graph's memory pool and are handed out again.  Holding all of them alive gave the row gathers 16 - 24
            # distinct 134 MB outputs next to 4 GB of tables and cost them 7 - 14 % (address translation, not
            # bandwidth: the same launches one at a time behind a cache flush take the same time wherever the
            # buffers lie).
            held = collections.deque(maxlen=copies if keep is None else keep)
            for _ in range(rounds):
                for p in pool:
                    held.append(fn(*p, **kwargs))
        run, per_run, how = graph.replay, launches, f"hip graph of {launches} launches over {copies} input copies, events around replays"
    except Exception as exc:  # noqa: BLE001
        print(f"measure: graph capture failed for this op ({exc}); eager launches", file=sys.stderr)
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




def calib_block(dev):
    """What this chip, in this run, sustains - so that a row's fraction of the nominal peak can be read
    against a ceiling measured in the same process:
      copy      the library's plain copy kernel, 128 MiB -> 128 MiB, timed like a per-op row;
      copy_fit  its time over five sizes, least-squares line t = intercept + bytes / asymptote: what a
                memory-bound row of a given size can at best be expected to take (launch ramp included);
      mfma      the GEMM kernels' matrix-core instruction streams with no memory traffic in the loop
                (mi355_calib_mfma): the 16x16x32 stream of the large-tile kernel (variant 10) and the 32x32x16
                stream (variant 0), on operands drawn like the GEMM rows' and on zeros.  The gap between the two
                fills is the power / clock envelope, the gap between zeros and 2.5 PFLOP/s the issue rate."""
    import torch

    from backendbench_amd.ops._common import copy_into

    cache = {}
    sizes = [16, 32, 64, 128, 256]  # MiB moved in total (half read, half written)
    ms = [copy_ms_for(mb << 20, dev, cache) for mb in sizes]
    n = len(sizes)
    xs = [float(mb << 20) for mb in sizes]
    mx, my = sum(xs) / n, sum(ms) / n
    slope = sum((x - mx) * (y - my) for x, y in zip(xs, ms)) / sum((x - mx) ** 2 for x in xs)  # ms per byte
    intercept = my - slope * mx
    big = ms[sizes.index(256)]
    out = {
        "copy": {"bytes": 256 << 20, "ms": round(big, 5), "gbs": round((256 << 20) / (big * 1e-3) / 1e9, 1),
                 "frac": round((256 << 20) / (big * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        "copy_fit": {"mib_moved": sizes, "ms": [round(v, 5) for v in ms], "intercept_us": round(intercept * 1e3, 3),
                     "asymptote_gbs": round(1.0 / slope / 1e6, 1), "asymptote_frac": round(1.0 / slope / 1e6 / HBM_PEAK_GBS, 4)},
        "mfma": {},
    }
    for name, variant, fill in (("x16_stream_gemm_data", 10, None), ("x16_stream_zeros", 10, "zeros"),
                                ("x32_stream_gemm_data", 0, None), ("x32_stream_zeros", 0, "zeros")):
        r = calib_mfma(dev, fill, variant)
        out["mfma"][name] = {"variant": variant, "tflops": r["tflops"], "frac_of_peak": r["frac_of_peak"]}
    torch.cuda.empty_cache()
    return out


def _gpt2_small(dev, dt, vocab=50257, width=768, layers=12, heads=12, positions=1024):
    """GPT-2 small as plain torch modules (token + position embedding, 12 pre-norm blocks of causal
    self-attention and a 4x GELU MLP, final layer norm, tied-shape vocabulary projection), randomly initialised.
    Written out here so that nothing in the forward pass depends on the host (no data-dependent Python branches,
    no .item()): the same call can be recorded into a HIP graph."""
    import torch
    from torch import nn

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.ln1, self.ln2 = nn.LayerNorm(width), nn.LayerNorm(width)
            self.qkv, self.proj = nn.Linear(width, 3 * width), nn.Linear(width, width)
            self.fc1, self.fc2 = nn.Linear(width, 4 * width), nn.Linear(4 * width, width)

        def forward(self, x, mask):
            B, T, C = x.shape
            q, k, v = self.qkv(self.ln1(x).view(B * T, C)).view(B, T, 3, heads, C // heads).permute(2, 0, 3, 1, 4)
            att = torch.matmul(q, k.transpose(-1, -2)) * (1.0 / (C // heads) ** 0.5)
            att = torch.softmax(att + mask, dim=-1)
            y = torch.matmul(att, v).transpose(1, 2).reshape(B * T, C)
            x = x + self.proj(y).view(B, T, C)
            h = torch.nn.functional.gelu(self.fc1(self.ln2(x).view(B * T, C)), approximate="tanh")
            return x + self.fc2(h).view(B, T, C)

    class GPT2(nn.Module):
        def __init__(self):
            super().__init__()
            self.wte, self.wpe = nn.Embedding(vocab, width), nn.Embedding(positions, width)
            self.blocks = nn.ModuleList(Block() for _ in range(layers))
            self.ln_f = nn.LayerNorm(width)
            self.head = nn.Linear(width, vocab, bias=False)

        def forward(self, ids, pos, mask):
            x = self.wte(ids) + self.wpe(pos)
            for blk in self.blocks:
                x = blk(x, mask)
            B, T, C = x.shape
            return self.head(self.ln_f(x).view(B * T, C)).view(B, T, -1)

    torch.manual_seed(0)
    model = GPT2()
    for p in model.parameters():
        if p.dim() > 1:
            nn.init.normal_(p, std=0.02)
    return model.to(device=dev, dtype=dt).eval()


def e2e_gpt2(dev, dtype_name="bf16", batch=8, seq=1024, reps=10):
    """One forward pass of a randomly initialised GPT-2 small (12 layers, 768 wide, 12 heads, 50257-token
    vocabulary) on `batch` x `seq` tokens: ms per forward with this backend's kernels behind the dispatcher
    (enable()) and with the stock ROCm kernels, launched eagerly from Python and replayed from a HIP graph.
    Eager rows also give the host's share: the time the Python thread needs to enqueue one forward (no device
    sync inside), which bounds the eager rate from below whenever it exceeds the GPU time.  The reference quotes
    this kind of figure for its own kernels (docs/correctness.md:21: "about twice as slow as PyTorch eager")."""
    import torch

    import backendbench_amd

    dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype_name]
    model = _gpt2_small(dev, dt)
    ids = torch.randint(0, 50257, (batch, seq), generator=torch.Generator().manual_seed(1)).to(dev)
    pos = torch.arange(seq, device=dev).unsqueeze(0)
    mask = torch.full((seq, seq), float("-inf"), device=dev, dtype=dt).triu(1)   # additive causal mask, built once

    def forward():
        with torch.no_grad():
            return model(ids, pos, mask)

    def timed(run, n):
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(n):
            run()
        e1.record()
        host = (time.perf_counter() - t0) * 1e3 / n       # enqueue only: nothing waits for the device in the loop
        torch.cuda.synchronize()
        return {"ms_per_forward": round(e0.elapsed_time(e1) / n, 3), "host_enqueue_ms": round(host, 3)}

    def both_modes():
        out = {"eager": timed(forward, reps)}
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):     # warm-up on the capture's kind of stream: lazy set-up happens here
                forward()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                held = forward()
            out["graph"] = timed(graph.replay, reps)
            del held, graph
        except Exception as exc:  # noqa: BLE001
            out["graph"] = {"error": str(exc)[:300]}
            torch.cuda.synchronize()
        return out

    ref = forward().float()
    stock = both_modes()
    kernel_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "generated_kernels")
    with backendbench_amd.BackendBench.enable(kernel_dir=kernel_dir, dispatch_key="CUDA"):
        got = forward().float()
        ours = both_modes()
        torch.cuda.synchronize()
    err = float((got - ref).abs().max()) / max(float(ref.abs().max()), 1e-6)
    res = {"only_op": "e2e.gpt2", "model": "GPT-2 small (12 x 768, 12 heads, vocabulary 50257), random weights", "dtype": dtype_name,
           "tokens": [batch, seq], "stock": stock, "override": ours, "max_abs_diff_of_logits_over_scale": round(err, 5)}
    for mode in ("eager", "graph"):
        a, b = stock[mode].get("ms_per_forward"), ours[mode].get("ms_per_forward")
        if a and b:
            res[f"speedup_{mode}"] = round(a / b, 3)
    return res


def only_op(args, backend, by_key, dev):
    """`bench.py --only-op <row>` and its diagnostic forms; prints one JSON line."""
    import torch

    if args.only_op == "calib.mfma":
        print(json.dumps(calib_mfma_f64(dev, args.variant or 16) if args.dtype == "f64" else calib_mfma(dev, args.fill, args.variant)))
        return
    if args.only_op == "e2e.gpt2":
        print(json.dumps(e2e_gpt2(dev, args.dtype if args.dtype in ("bf16", "f16", "f32") else "bf16")))
        return
    if args.only_op == "calib.all":
        print(json.dumps({"only_op": "calib.all", **calib_block(dev)}))
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
    if args.trace:
        print(json.dumps(gemm_trace(by_key[args.only_op], dev, args.fill)))
        return
    if args.ablate is not None:
        print(json.dumps(gemm_ablate(by_key[args.only_op], dev, args.ablate, args.fill)))
        return
    if args.only_op == "calib.copy":
        from backendbench_amd.ops._common import copy_into

        src = torch.empty(32 * 2**20, dtype=torch.float32, device=dev).normal_()
        f, a, kw, work = (lambda s: copy_into(torch.empty_like(s), s)), [src], {}, 2 * src.numel() * 4
    else:
        case = by_key[args.only_op]
        a, kw = case.make(dev)
        f, work = backend[case.op], case.work
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
