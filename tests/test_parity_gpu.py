"""Parity of the HIP kernels with the oracle (ATen on CPU, oracle/aten_cpu.py) on identical
seeded inputs, through the drop-in boundary: DirectoryBackend -> `<folder>_kernel_impl` ->
ctypes -> libmi355_aten.so.

Bar: bit-exact for integer / index / copy outputs (argmax, gather, index_select, embedding,
where, integer arithmetic); atol = rtol = 1e-2 with NaN == NaN for floating point — the only
tolerance the reference enforces (BackendBench/eval.py:68-90) — dtype and shape included.
"""

import os
import sys

import pytest
import torch

from backendbench_amd import eval as ev
from backendbench_amd.backends import DirectoryBackend
from backendbench_amd.suite import SmokeTestSuite, edge_cases, perf_cases
from oracle import aten_cpu

from tight import tight_check  # noqa: E402

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
aten = torch.ops.aten
EDGE = edge_cases()
PERF = perf_cases()


@pytest.fixture(scope="module")
def backend():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    b = DirectoryBackend(os.path.join(ROOT, "generated_kernels"))
    assert len(b.compiled_kernels) == 68
    return b


def announce(what):
    print(f"\n[gpu-case] {what}", flush=True)
    sys.stdout.flush()


def run_case(backend, case):
    announce(case.key)
    args, kwargs = case.make("cuda")
    res = backend[case.op](*args, **kwargs)
    torch.cuda.synchronize()
    from backendbench_amd.ops import check_index_errors

    check_index_errors()
    ref = aten_cpu.reference(case.op, args, kwargs)
    res_cpu = aten_cpu.to_cpu(res)
    for r in (res if isinstance(res, (tuple, list)) else [res]):
        assert r.device.type == "cuda"
    ok = ev.allclose(ref, res_cpu, exact=case.exact)
    if not ok:
        a, r = ev.compute_errors(ref, res_cpu)
        pytest.fail(f"{case.key}: mismatch (max abs {a}, max rel {r}); ref={ref!r:.400} res={res_cpu!r:.400}")
    # the second, per-dtype bar: against the numpy float64 restatement (tests/tight.py)
    msg = tight_check(case, aten_cpu.to_cpu(list(args)), aten_cpu.to_cpu(dict(kwargs)), res_cpu)
    assert msg is None, f"{case.key}: {msg}"


@pytest.mark.parametrize("case", EDGE, ids=[c.key for c in EDGE])
def test_edge_case_parity(backend, case):
    run_case(backend, case)


SMALL_PERF = [c for c in PERF if not c.key.startswith(("C3.", "C4.argmax", "C4.embedding", "C4.index_select"))]


@pytest.mark.parametrize("case", SMALL_PERF, ids=[c.key for c in SMALL_PERF])
def test_headline_shape_parity(backend, case):
    """Full BASELINE shapes the CPU oracle finishes in seconds: compared element by element."""
    run_case(backend, case)


def test_headline_indexing_full_size(backend):
    """embedding / index_select at [128256, 4096] bf16 with 16384 indices: bit-exact against
    the oracle, plus the identities embedding == index_select(0) and out[j] == table[idx[j]]."""
    announce("C4.embedding/index_select full size")
    case = next(c for c in PERF if c.key == "C4.embedding")
    (table, idx), _ = case.make("cuda")
    emb = backend[aten.embedding.default](table, idx)
    sel = backend[aten.index_select.default](table, 0, idx)
    torch.cuda.synchronize()
    assert ev.bit_equal(emb, sel)
    ref = aten_cpu.reference(aten.embedding.default, [table, idx])
    assert ev.bit_equal(ref, emb.cpu())
    perm = torch.randperm(table.shape[0], generator=torch.Generator().manual_seed(0)).cuda()
    assert ev.bit_equal(backend[aten.index_select.default](table, 0, perm)[torch.argsort(perm)], table)  # round trip


def test_headline_argmax_full_size(backend):
    """argmax over fp32 [8192, 128256] (4.2 GB): bit-exact against the oracle; amax agrees
    with a gather at the argmax; planted ties and NaNs resolve to the first index."""
    announce("C4.argmax full size")
    case = next(c for c in PERF if c.key == "C4.argmax")
    (x, dim), _ = case.make("cuda")
    x[5, 1000] = x[5, 77] = 9.0            # tie: first wins
    x[6, 128255] = float("nan")            # NaN is the maximum
    x[7, 3] = x[7, 2] = float("nan")
    x[8, :] = -float("inf")
    got = backend[aten.argmax.default](x, dim)
    torch.cuda.synchronize()
    assert got.dtype == torch.int64 and got.shape == (x.shape[0],)
    assert got[5].item() == 77 and got[6].item() == 128255 and got[7].item() == 2 and got[8].item() == 0
    ref = aten_cpu.reference(aten.argmax.default, [x, dim])
    assert torch.equal(ref, got.cpu())
    mx = backend[aten.amax.default](x[:4096], [-1])
    picked = backend[aten.gather.default](x[:4096], 1, got[:4096, None]).squeeze(1)
    assert ev.bit_equal(mx, picked)


@pytest.mark.parametrize("key", ["C3.mm_up", "C3.addmm_up", "C3.mm_down", "C3.addmm_down"])
def test_headline_gemm_full_size(backend, key):
    """7B-MLP GEMMs at full size: the whole [4096, N] product against the oracle (ATen on the
    host CPU runs one of these in about a tenth of a second), then linearity in alpha."""
    announce(key)
    case = next(c for c in PERF if c.key == key)
    args, kwargs = case.make("cuda")
    out = backend[case.op](*args, **kwargs)
    torch.cuda.synchronize()
    ref = aten_cpu.reference(case.op, args, kwargs)
    got = out.cpu()
    assert got.shape == ref.shape and got.dtype == ref.dtype
    assert ev.allclose(ref, got), ev.compute_errors(ref, got)
    assert torch.isfinite(got.float()).all()
    if "addmm" in key:
        doubled = backend[case.op](*args, alpha=2.0, beta=0.0)
        plain = backend[aten.mm.default](args[1], args[2])
        assert ev.allclose((2 * plain.float()).to(plain.dtype).cpu(), doubled.cpu())


@pytest.mark.parametrize("waves", ["4", "8", "256x128"])
@pytest.mark.parametrize("layout", ["nt", "nn", "tn", "tt"])
def test_large_tile_gemm_every_k_loop_length(backend, layout, waves, gemm_knobs):
    """The 256x256-tile kernels only run when a problem has enough tiles to fill the chip, so the
    small K-step cases of the edge suite never reach them.  A [3500, K] x [K, 3600] product has
    14 x 15 tiles (ragged last row and column of tiles); K walks through every prologue / steady /
    drain length of the 64-k pipelines, the 32-k ring (K % 64 == 32) and the zero-filled K tail.
    Small-integer operands make the fp32 accumulation exact, so the sampled rows must be
    bit-equal to the oracle's.  MI355_GEMM_WAVES forces one of the two 64-k kernels (eight waves of
    128x64 or four of 128x128), which otherwise split the K range between them; MI355_GEMM_TILE
    forces the four-wave kernel on 256x128 tiles for every K that is a multiple of 64."""
    announce(f"large-tile GEMM K loop lengths, {layout}, {waves}")
    if waves == "256x128":   # the four-wave kernel on 256x128 tiles, otherwise chosen for mid-sized problems
        gemm_knobs.tile(waves)
    else:
        gemm_knobs.waves(waves)
    g = torch.Generator().manual_seed(5)
    M, N = (3504, 3600) if layout[0] == "t" else (3500, 3600)   # an M-contiguous operand needs M % 8 == 0
    rows = torch.unique(torch.cat([torch.randint(0, M, (40,), generator=g), torch.tensor([0, 127, 128, 255, 256, 3327, 3328, 3499])]))
    for K in (64, 128, 192, 256, 320, 384, 448, 512, 576, 640, 704, 1024, 2048, 2112, 96, 160, 288, 72, 200):
        if layout[0] == "t":   # transposed left operand (M-contiguous): taken as it is when K % 64 == 0
            a = torch.randint(-1, 2, (K, M), generator=g).to(torch.bfloat16).cuda().t()
        else:
            a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
        if layout[1] == "t":
            b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
        else:
            b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).cuda()
        out = backend[aten.mm.default](a, b)
        ref = aten_cpu.reference(aten.mm.default, [a[rows.cuda()], b])
        assert ev.bit_equal(ref, out[rows.cuda()].cpu()), (layout, K)
        bias = torch.randint(-2, 3, (N,), generator=g).to(torch.bfloat16).cuda()
        out2 = backend[aten.addmm.default](bias, a, b)
        assert ev.bit_equal((out.float() + bias.float()).to(torch.bfloat16), out2), (layout, K, "bias")


@pytest.mark.parametrize("layout", ["nt", "nn", "tn", "tt"])
def test_mixed_width_tile_grid(backend, layout, gemm_knobs):
    """More than one round of 256x256 tiles with a ragged last round: the four-wave kernel cuts the last
    columns into 192-wide tiles (one launch, two tile widths).  [4104, K] x [K, 4500] has 17 x 18 tiles of
    256x256; the planner must choose a mixed grid for it, the result must be bit-equal to the plain grid's
    (same k order per element) and, on small-integer operands, to the oracle's on sampled rows.  Covers the
    ragged last tile row, the ragged last (narrow) tile column and every K-loop length of the kernel."""
    import ctypes

    from backendbench_amd import _lib
    announce(f"mixed-width tile grid, {layout}")
    M, N = 4104, 4500
    wide, narrow = ctypes.c_int32(), ctypes.c_int32()
    assert _lib.load().mi355_gemm_tile_columns(M, N, 4096, ctypes.byref(wide), ctypes.byref(narrow)) == 0
    assert narrow.value > 0, "this shape is meant to take the mixed grid"
    gemm_knobs.waves("4")
    g = torch.Generator().manual_seed(11)
    edge = wide.value * 256
    rows = torch.unique(torch.cat([torch.randint(0, M, (40,), generator=g), torch.tensor([0, 255, 256, 4095, 4096, 4103])]))
    for K in (64, 128, 192, 256, 320, 384, 448, 512, 576, 1024, 2112, 4096):
        if layout[0] == "t":
            a = torch.randint(-1, 2, (K, M), generator=g).to(torch.bfloat16).cuda().t()
        else:
            a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
        if layout[1] == "t":
            b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
        else:
            b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).cuda()
        bias = torch.randint(-2, 3, (N,), generator=g).to(torch.bfloat16).cuda()
        gemm_knobs.tile("mixed")      # the mixed grid whatever K is (by itself: K >= 4096)
        mixed = backend[aten.addmm.default](bias, a, b)
        gemm_knobs.tile("256x256")
        plain = backend[aten.addmm.default](bias, a, b)
        gemm_knobs.tile(None)
        assert ev.bit_equal(plain, mixed), (layout, K)
        ref = aten_cpu.reference(aten.addmm.default, [bias, a[rows.cuda()], b])
        assert ev.bit_equal(ref, mixed[rows.cuda()].cpu()), (layout, K)
        assert ev.bit_equal(ref[:, edge - 8:edge + 200], mixed[rows.cuda()][:, edge - 8:edge + 200].cpu())  # across the seam


@pytest.mark.parametrize("layout", ["nt", "nn"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_split_k_inside_one_launch(backend, layout, dtype, gemm_knobs):
    """Products with 65 - 128 tiles of 256x256 and K >= 2048 (1536 for 96 - 112 tiles, 3072 above): two workgroups per tile take about half of K each, one
    leaves its fp32 accumulators in the workspace and raises a flag, the other adds them to its own and runs
    the epilogue.  Tile counts at both ends of the range and off the multiples of 8, ragged last tile rows and
    columns, output rows off the 128-byte lines and (transposed b) off the 16-byte units, unit counts of K
    that do not halve, plain / bias row / full c epilogues.  Small-integer operands make the two-part sum
    exact: bit-equal to the oracle.  A HIP graph of such products is replayed with eager work in between -
    the flags must be back at zero after every run, whoever used the workspace memory in the meantime."""
    import ctypes

    from backendbench_amd import _lib
    announce(f"GEMM split K inside one launch, {layout}, {dtype}")
    lib = _lib.load()
    g = torch.Generator().manual_seed(31)
    shapes = [(2048, 3072, 2304), (2100, 3200, 2500), (3584, 3072, 2048 + 8), (1536, 4224, 2816), (1000, 3072, 5000),
              (2048, 2048, 2304), (2100, 2176, 2500),          # (K at the lower bound; 17 units of K)
              (2048, 1536, 3072)]                              # (96 - 112 tiles: from K = 1536)
    if layout == "nt":
        shapes += [(1792, 3072, 4097), (2304, 3456, 2818)]
    # three and four workgroups per tile (the summing one then reads two or three planes): a knob, at any tile count
    forced = [("x16split3", 1536, 3200, 1024 + 8), ("x16split4", 700, 4096, 1280), ("x16split4", 2048, 2048 + 128, 2304)]
    for knob, M, K, N in [(None, *sh) for sh in shapes] + forced:
        tiles = -(-M // 256) * -(-N // 256)
        gemm_knobs.tile(knob)
        parts = int(knob[-1]) if knob else 2
        assert knob is not None or 64 < tiles <= 128, (M, N, tiles)
        assert lib.mi355_gemm_workspace_bytes(M, N, K, _lib.dtype_code(dtype)) >= (parts - 1) * tiles * (256 * 256 * 4 + 8)
        # one in four entries of a is non-zero: every |sum| stays far below 256, exact in bf16 as well
        a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.randint(0, 4, (M, K), generator=g) == 0)).to(dtype).cuda()
        if layout == "nt":
            b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t()
        else:
            b = torch.randint(-1, 2, (K, N), generator=g).to(dtype).cuda()
        bias = torch.randint(-2, 3, (N,), generator=g).to(dtype).cuda()
        full = torch.randint(-2, 3, (M, N), generator=g).to(dtype).cuda()
        # the oracle on the fp32 copies (its f16 kernel takes a minute here): exact integer sums, exact in `dtype`
        ref = aten_cpu.reference(aten.mm.default, [a.float(), b.float()])
        assert float(ref.abs().max()) <= 192
        ref = ref.to(dtype)
        out = backend[aten.mm.default](a, b)
        assert ev.bit_equal(ref, out.cpu()), (layout, M, K, N)
        out = backend[aten.addmm.default](bias, a, b)
        assert ev.bit_equal((ref.float() + bias.cpu().float()).to(dtype), out.cpu()), (layout, M, K, N, "bias row")
        out = backend[aten.addmm.default](full, a, b, beta=2, alpha=0.5)
        assert ev.bit_equal((0.5 * ref.float() + 2 * full.cpu().float()).to(dtype), out.cpu()), (layout, M, K, N, "full c")
    gemm_knobs.tile(None)
    # graph replays: the same launches (same flag value) on the same workspace memory, run after run
    M, K, N = shapes[1]
    a = torch.randint(-1, 2, (M, K), generator=g).to(dtype).cuda()
    b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t() if layout == "nt" else torch.randint(-1, 2, (K, N), generator=g).to(dtype).cuda()
    a2 = torch.randint(-1, 2, (M, K), generator=g).to(dtype).cuda()
    want, want2 = backend[aten.mm.default](a, b), backend[aten.mm.default](a2, b)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = backend[aten.mm.default](a, b)
        got2 = backend[aten.mm.default](a2, b)
    for rep in range(4):
        got.zero_()
        got2.zero_()
        junk = torch.full((64 << 20,), float(rep), device="cuda")   # eager work that may land on the freed workspace
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert ev.bit_equal(want, got) and ev.bit_equal(want2, got2), (layout, "replay", rep)
        del junk


@pytest.mark.parametrize("form", ["planner", "x16", "x16mixed", "256x128", "mixed", "w4", "w8", "64x64", "128x128"])
def test_gemm_output_rows_off_16_byte_boundaries(backend, form, gemm_knobs):
    """An output width that is no multiple of 8 (a 50257-wide vocabulary) puts every row of the result at
    another 2-byte offset; the MFMA kernels then store along the destination's 16-byte grid: whole units
    inside a tile's row segment, single elements at its two ends (those units are shared with the
    neighbouring tile's columns).  Every residue of N mod 8 (and two widths that are multiples of 8 but not
    of 64: rows on 16-byte boundaries off the 128-byte lines), ragged last tile rows and columns, each
    kernel form (forced by its knob), with and without a bias row.  Small-integer operands: bit-equal to
    the oracle.  The C entry point is also handed an output one element into a larger buffer, whose
    guard elements in front and behind must come back untouched."""
    from backendbench_amd import _lib
    from backendbench_amd.ops._common import launch
    announce(f"GEMM output rows off 16-byte boundaries, {form}")
    if form in ("w4", "w8"):
        gemm_knobs.waves(form[1])
    elif form != "planner":
        gemm_knobs.tile(form)
        if form == "mixed":   # the mixed-width grid belongs to the four-wave 32x32x16 kernel
            gemm_knobs.waves("4")
    g = torch.Generator().manual_seed(23)
    M, K = (1000, 256) if form in ("64x64", "128x128") else (2300, 256)
    widths = (257, 1026, 1283, 2052, 2309, 2566, 2823, 301) if form in ("64x64", "128x128") else (4097, 4098, 4355, 4100, 4613, 4358, 4103, 4104, 4376)
    a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
    for N in widths:
        b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
        bias = torch.randint(-2, 3, (N,), generator=g).to(torch.bfloat16).cuda()
        ref = aten_cpu.reference(aten.mm.default, [a, b])
        out = backend[aten.mm.default](a, b)
        assert ev.bit_equal(ref, out.cpu()), (form, N)
        out2 = backend[aten.addmm.default](bias, a, b)
        assert ev.bit_equal((ref.float() + bias.cpu().float()).to(torch.bfloat16), out2.cpu()), (form, N, "bias")
        # one element into the storage (rows at every 2-byte offset, guard elements around the result)
        big = torch.full((M * N + 64,), 77.0, dtype=torch.bfloat16, device="cuda")
        view = big[33:33 + M * N].view(M, N)
        launch("mi355_gemm", a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), None, 0, 0,
               view.data_ptr(), M, N, K, 1.0, 0.0, _lib.dtype_code(a.dtype), None, 0)
        assert ev.bit_equal(ref, view.cpu()), (form, N, "offset view")
        assert bool((big[:33] == 77.0).all()) and bool((big[33 + M * N:] == 77.0).all()), (form, N, "guard elements")


@pytest.mark.parametrize("tile", ["x16", "x16mixed", "planner"])
@pytest.mark.parametrize("layout", ["nt", "nn"])
def test_x16_gemm_every_k_loop_length(backend, layout, tile, gemm_knobs):
    """The 256x256-tile kernel on v_mfma_f32_16x16x32 (the planner's choice for products that fill the chip
    when K is a multiple of 128 from 512 on): [4104, K] x [K, 4500] has 17 x 18 tiles with a ragged last tile
    row and column; K walks from the shortest loop the kernel takes (two pairs of stages: only the peeled
    end of the pipeline) through every count of steady-state iterations up to 4096.  MI355_GEMM_TILE=x16
    forces the kernel for every K, =x16mixed its two-width grid (192-wide tiles behind the 256-wide ones:
    the seam is checked), and "planner" leaves the choice to the library.  Small-integer operands make the
    fp32 accumulation exact, so sampled rows must be bit-equal to the oracle's; a bias row and an f16 run go
    through the same epilogue."""
    import ctypes

    from backendbench_amd import _lib
    announce(f"16x16x32 GEMM K loop lengths, {layout}, {tile}")
    M, N = 4104, 4500
    wide, narrow = ctypes.c_int32(), ctypes.c_int32()
    assert _lib.load().mi355_gemm_tile_columns(M, N, 4096, ctypes.byref(wide), ctypes.byref(narrow)) == 0
    assert narrow.value > 0
    edge = wide.value * 256
    g = torch.Generator().manual_seed(13)
    rows = torch.unique(torch.cat([torch.randint(0, M, (40,), generator=g), torch.tensor([0, 63, 64, 127, 128, 255, 256, 4095, 4096, 4103])]))
    for K in (256, 384, 512, 640, 768, 896, 1024, 1152, 1280, 2048, 4096):
        a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
        if layout[1] == "t":
            b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
        else:
            b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).cuda()
        bias = torch.randint(-2, 3, (N,), generator=g).to(torch.bfloat16).cuda()
        if tile != "planner":
            gemm_knobs.tile(tile)
        out = backend[aten.addmm.default](bias, a, b)
        half = backend[aten.mm.default](a.half(), b.half())
        if tile != "planner":
            gemm_knobs.tile(None)
        ref = aten_cpu.reference(aten.addmm.default, [bias, a[rows.cuda()], b])
        assert ev.bit_equal(ref, out[rows.cuda()].cpu()), (layout, tile, K)
        assert ev.bit_equal(ref[:, edge - 8:edge + 200], out[rows.cuda()][:, edge - 8:edge + 200].cpu()), (layout, tile, K, "seam")
        ref16 = aten_cpu.reference(aten.mm.default, [a.half()[rows.cuda()], b.half()])
        assert ev.bit_equal(ref16, half[rows.cuda()].cpu()), (layout, tile, K, "f16")


@pytest.mark.parametrize("tile", ["x16", "x16persist"])
def test_x16_gemm_argument_forms(backend, tile, gemm_knobs):
    """What else reaches the 16x16x32 kernel besides dense operands: rows with a pitch (slices of wider tensors) on
    both operands, a c that is a column ([M, 1]), a scalar-strided c (a transposed view), a c of NaNs under beta = 0
    (never read), alpha and beta other than one, f16.  [512, 640] x [640, 768]: 2 x 3 tiles, forced onto the kernel
    (one workgroup per tile, and the persistent walk).  Small-integer operands: bit-equal to the oracle."""
    announce(f"16x16x32 GEMM argument forms, {tile}")
    g = torch.Generator().manual_seed(15)
    M, K, N = 512, 640, 768
    ri = lambda *s, lo=-1, hi=2: torch.randint(lo, hi, s, generator=g)  # noqa: E731
    for dtype in (torch.bfloat16, torch.float16):
        wide_a = ri(M, K + 64).to(dtype).cuda()
        wide_b = ri(K, N + 128).to(dtype).cuda()
        wide_bt = ri(N, K + 8).to(dtype).cuda()
        a = wide_a[:, 32:32 + K]            # 64-byte offset, pitch K + 64
        b = wide_b[:, 64:64 + N]
        bt = wide_bt[:, :K].t()
        col = ri(M, 1, lo=-2, hi=3).to(dtype).cuda()
        full_t = ri(N, M, lo=-2, hi=3).to(dtype).cuda().t()
        nan_c = torch.full((M, N), float("nan"), dtype=dtype).cuda()
        gemm_knobs.tile(tile)
        outs = {
            "pitched nn": (backend[aten.mm.default](a, b), aten.mm.default, [a, b], {}),
            "pitched nt": (backend[aten.mm.default](a, bt), aten.mm.default, [a, bt], {}),
            "column c": (backend[aten.addmm.default](col, a, b), aten.addmm.default, [col, a, b], {}),
            "transposed c": (backend[aten.addmm.default](full_t, a, bt, beta=2.0, alpha=3.0), aten.addmm.default, [full_t, a, bt], {"beta": 2.0, "alpha": 3.0}),
            "nan c, beta 0": (backend[aten.addmm.default](nan_c, a, b, beta=0.0, alpha=2.0), aten.addmm.default, [nan_c, a, b], {"beta": 0.0, "alpha": 2.0}),
        }
        gemm_knobs.tile(None)
        for name, (got, op, args, kwargs) in outs.items():
            ref = aten_cpu.reference(op, args, kwargs)
            assert ev.bit_equal(ref, got.cpu()), (tile, dtype, name)


@pytest.mark.parametrize("layout", ["nt", "nn"])
def test_x16_persistent_gemm_walks_its_tiles(backend, layout, gemm_knobs):
    """More 256x256 tiles than CUs: one workgroup per CU walks its tiles, with the fill requests running on
    from one tile into the next.  [4096, K] x [K, 4352] has 16 x 17 = 272 tiles (sixteen workgroups get a second
    tile), [2048, K] x [K, 12288] 8 x 48 = 384 (half of them), [256, K] x [K, 256] a single one (forced: a walk
    of one tile).  K from the shortest loop the walk takes (384: the four special half-stages and the eight last
    ones, no steady iteration) upwards.  Bit-equal to the one-workgroup-per-tile form of the same kernel
    (same k order per element) and, on small-integer operands, to the oracle on sampled rows; bias row and a
    full c through the epilogue's four passes."""
    from backendbench_amd import _lib
    from backendbench_amd.ops._common import launch
    announce(f"persistent 16x16x32 GEMM, {layout}")
    g = torch.Generator().manual_seed(14)
    # (4000, 4416), (2100, 12352), (300, 320): M and N off the multiples of 256 (N a multiple of 64) - the walk moves
    # its last row / column of tiles back to the matrix edge and stores the overlap twice
    for (M, N) in ((4096, 4352), (2048, 12288), (256, 256), (4000, 4416), (2100, 12352), (300, 320)):
        rows = torch.unique(torch.cat([torch.randint(0, M, (24,), generator=g), torch.tensor([0, 63, 64, 127, 128, 255, M - 1])]))
        for K in (384, 512, 640, 768, 1024, 2048):
            a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
            if layout[1] == "t":
                b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
            else:
                b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).cuda()
            bias = torch.randint(-2, 3, (N,), generator=g).to(torch.bfloat16).cuda()
            c = torch.randint(-2, 3, (M, N), generator=g).to(torch.bfloat16).cuda()
            gemm_knobs.tile("x16persist")
            walked = backend[aten.addmm.default](bias, a, b)
            walked_c = backend[aten.addmm.default](c, a, b, beta=2.0)
            walked_mm = backend[aten.mm.default](a, b)
            gemm_knobs.tile("x16")
            plain = backend[aten.addmm.default](bias, a, b)
            gemm_knobs.tile(None)
            auto = backend[aten.addmm.default](bias, a, b)
            assert ev.bit_equal(plain, walked), (layout, M, N, K)
            assert ev.bit_equal(plain, auto), (layout, M, N, K, "planner's choice")
            ref = aten_cpu.reference(aten.addmm.default, [bias, a[rows.cuda()], b])
            assert ev.bit_equal(ref, walked[rows.cuda()].cpu()), (layout, M, N, K)
            ref_c = aten_cpu.reference(aten.addmm.default, [c[rows.cuda()], a[rows.cuda()], b], {"beta": 2.0})
            assert ev.bit_equal(ref_c, walked_c[rows.cuda()].cpu()), (layout, M, N, K, "full c")
            assert ev.bit_equal((walked.float() - bias.float()).to(torch.bfloat16), walked_mm), (layout, M, N, K, "mm")
            if (M % 256 or N % 256) and K == 768:
                # c in the memory of out (the C entry point allows it): no element may take beta * c twice
                gemm_knobs.tile("x16persist")
                acc = c.clone()
                launch("mi355_gemm", a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), acc.data_ptr(), N, 1,
                       acc.data_ptr(), M, N, K, 1.0, 2.0, _lib.dtype_code(a.dtype), None, 0)
                gemm_knobs.tile(None)
                assert ev.bit_equal(walked_c, acc), (layout, M, N, K, "c in place")


@pytest.mark.parametrize("layout", ["nt", "nn", "tn", "tt"])
@pytest.mark.parametrize("shape", [(704, 900), (2000, 2500), (704, 900, "ring4"), (704, 900, "ring8")])
def test_small_tile_gemm_every_k_loop_length(backend, layout, shape, gemm_knobs):
    """The 128x128-tile kernels: [704, K] x [K, 900] has 6 x 8 tiles, at most one workgroup per CU
    (the deep-ring kernel when K is a multiple of 64, split along K once K is long enough for the
    planner); [2000, K] x [K, 2500] has 16 x 20, more than one per CU (the two-per-CU kernel).  K
    walks through every prologue / steady / drain length of both pipelines.  The deep-ring kernel has a
    four-wave form and one with four more waves that issue the fills; the planner picks by layout, and
    `ring4` / `ring8` force each on every layout.  Small-integer operands make the fp32 accumulation exact
    in any order, so the sampled rows must be bit-equal to the oracle's."""
    M, N = shape[:2]
    if len(shape) > 2:
        gemm_knobs.tile(shape[2])
    announce(f"small-tile GEMM K loop lengths, {layout}, {shape}")
    g = torch.Generator().manual_seed(6)
    rows = torch.unique(torch.cat([torch.randint(0, M, (40,), generator=g), torch.tensor([0, 63, 64, 127, 128, M - 129, M - 128, M - 1])]))
    for K in (32, 64, 96, 128, 160, 192, 224, 256, 320, 384, 448, 512, 576, 640, 704, 1056, 2080, 4096):
        if layout[0] == "t":   # transposed left operand (M-contiguous): taken as it is when K % 64 == 0
            a = torch.randint(-1, 2, (K, M), generator=g).to(torch.bfloat16).cuda().t()
        else:
            a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
        if layout[1] == "t":
            b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
        else:
            b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).cuda()
        out = backend[aten.mm.default](a, b)
        ref = aten_cpu.reference(aten.mm.default, [a[rows.cuda()], b])
        assert ev.bit_equal(ref, out[rows.cuda()].cpu()), (layout, shape, K)


@pytest.mark.parametrize("layout", ["nt", "nn"])
@pytest.mark.parametrize("shape", [(197, 776), (1000, 1080), (64, 64), (33, 4104)])
def test_tile64_gemm_every_k_loop_length(backend, layout, shape, gemm_knobs):
    """The 64x64-tile kernel (products whose 128x128 tiles would leave most CUs idle): [197, K] x [K, 776] has
    4 x 13 tiles with ragged last row and column (one workgroup per CU: the eight-stage ring), [1000, K] x
    [K, 1080] has 16 x 17 = 272 (more than one per CU: the four-stage ring).  K walks from one stage to more
    than twice the ring depth.  Small-integer operands: bit-equal to the oracle; a bias row through the
    epilogue; the kernel is forced so that every K takes it, and once left to the planner."""
    M, N = shape
    announce(f"64x64-tile GEMM K loop lengths, {layout}, {M}x{N}")
    g = torch.Generator().manual_seed(12)
    for K in (64, 128, 192, 256, 384, 448, 512, 576, 640, 1024, 1088, 2048):
        a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).cuda()
        if layout[1] == "t":
            b = torch.randint(-1, 2, (N, K), generator=g).to(torch.bfloat16).cuda().t()
        else:
            b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).cuda()
        bias = torch.randint(-2, 3, (N,), generator=g).to(torch.bfloat16).cuda()
        gemm_knobs.tile("64x64")
        out = backend[aten.addmm.default](bias, a, b, beta=2.0)
        half = backend[aten.mm.default](a.half(), b.half())
        gemm_knobs.tile(None)
        ref = aten_cpu.reference(aten.addmm.default, [bias, a, b], {"beta": 2.0})
        assert ev.bit_equal(ref, out.cpu()), (layout, shape, K)
        assert ev.bit_equal(aten_cpu.reference(aten.mm.default, [a.half(), b.half()]), half.cpu()), (layout, shape, K, "f16")
        auto = backend[aten.addmm.default](bias, a, b, beta=2.0)
        assert ev.bit_equal(ref, auto.cpu()), (layout, shape, K, "planner's choice")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_k_with_ragged_k(backend, dtype):
    """One-tile outputs split along K where K is not a multiple of the split length (K = 4000, 2720, 5216, 3104
    in parts of whole 32-k steps, plus K = 672 .. 1184 around the length from which a split pays, and a 100 x 70
    output): every split, the last one included, must cover its own k range exactly.  Small-integer operands:
    bit-equal to the oracle whatever the order of the partial sums."""
    from backendbench_amd import _lib
    announce(f"split-K with ragged K, {dtype}")
    for K in (4000, 2720, 5216):
        assert _lib.load().mi355_gemm_workspace_bytes(64, 64, K, _lib.dtype_code(dtype)) > 0   # the planner does split these
    g = torch.Generator().manual_seed(9)
    for M, N, K in [(64, 64, 672), (64, 64, 544), (64, 64, 416), (64, 64, 1184), (100, 70, 928), (64, 64, 4000), (64, 64, 2720),
                    (64, 64, 5216), (128, 64, 3104), (33, 64, 1696)]:
        for nt in (False, True):
            a = torch.randint(-1, 2, (M, K), generator=g).to(dtype).cuda()
            b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t() if nt else torch.randint(-1, 2, (K, N + (-N) % 8), generator=g).to(dtype).cuda()
            out = backend[aten.mm.default](a, b)
            ref = aten_cpu.reference(aten.mm.default, [a, b])
            assert ev.bit_equal(ref, out.cpu()), (M, N, K, nt)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_k_on_64x64_tiles(backend, dtype, gemm_knobs):
    """A handful of 64x64 tiles with a long K (one image's 197 tokens against a 3072 x 768 weight) split K in
    whole 64-k stages over the chip: blockIdx.y owns a k range, leaves its raw fp32 tile in its plane, and the
    summing launch applies alpha / beta / bias.  Stage counts that do not divide by the split count, ragged
    and odd-N outputs, both layouts of b, every epilogue; MI355_GEMM_TILE=64x64 forces the kernel where the
    planner would take another one.  Small-integer operands: bit-equal to the oracle."""
    announce(f"split-K on 64x64 tiles, {dtype}")
    g = torch.Generator().manual_seed(43)
    for forced in (False, True):
        if forced:
            gemm_knobs.tile("64x64")
        for M, N, K in [(197, 768, 3072), (128, 768, 3136), (16, 4096, 4096), (70, 1001, 2112), (256, 4096, 4032), (64, 520, 11008), (300, 200, 1088)]:
            for nt in (True, False):
                if not nt and N % 8:
                    continue
                a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.randint(0, 4, (M, K), generator=g) == 0)).to(dtype).cuda()
                b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t() if nt else torch.randint(-1, 2, (K, N), generator=g).to(dtype).cuda()
                bias = torch.randint(-2, 3, (N,), generator=g).to(dtype).cuda()
                full = torch.randint(-2, 3, (M, N), generator=g).to(dtype).cuda()
                ref = aten_cpu.reference(aten.mm.default, [a.float(), b.float()])   # exact integer sums (the f16 CPU kernel is slow)
                assert float(ref.abs().max()) <= 192
                ref = ref.to(dtype)
                assert ev.bit_equal(ref, backend[aten.mm.default](a, b).cpu()), (forced, M, N, K, nt)
                out = backend[aten.addmm.default](bias, a, b)
                assert ev.bit_equal((ref.float() + bias.cpu().float()).to(dtype), out.cpu()), (forced, M, N, K, nt, "bias row")
                out = backend[aten.addmm.default](full, a, b, beta=2, alpha=0.5)
                assert ev.bit_equal((0.5 * ref.float() + 2 * full.cpu().float()).to(dtype), out.cpu()), (forced, M, N, K, nt, "full c")


@pytest.mark.parametrize("meet", ["inlaunch", "launch2", "inlaunch-ring4", "inlaunch-ring8", "launch2-ring8"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_k_parts_meet_either_way(backend, dtype, meet, gemm_knobs):
    """The parts of a K split on the 128x128- and 64x64-tile kernels meet in a summing launch or inside the one
    launch (the last part polls the others' flags, adds their planes and runs the epilogue): the planner picks
    per shape, the gemm_split knob forces one.  Shapes for the 64x64 tiles, the two-per-CU and the deep-ring 128x128
    kernels, part counts from 2 to dozens, ragged tiles and K ranges, both layouts of b, the three epilogues.
    Small-integer operands: bit-equal to the oracle either way.  Then a HIP graph of in-launch products is replayed
    with eager work in between: the flags must be back at zero after every run."""
    from backendbench_amd import _lib
    announce(f"split-K parts meet {meet}, {dtype}")
    lib = _lib.load()
    meet, _, ring = meet.partition("-")  # -ring4 / -ring8: one form of the deep-ring 128x128 kernel on both layouts (and no 64x64 tiles)
    gemm_knobs.split(meet)
    if ring:
        gemm_knobs.tile(ring)
    g = torch.Generator().manual_seed(47)
    shapes = [(1024, 2048, 4096), (1024, 2048, 4160), (512, 768, 3072), (197, 768, 3072), (128, 4096, 4096), (64, 64, 4000),
              (100, 70, 928), (1000, 1752, 2112), (256, 1024, 8192), (16, 4096, 4096), (700, 900, 2048)]
    split_seen = 0
    for M, N, K in shapes:
        split_seen += lib.mi355_gemm_workspace_bytes(M, N, K, _lib.dtype_code(dtype)) > 0
        for nt in (True, False):
            if not nt and N % 8:
                continue
            a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.randint(0, 4, (M, K), generator=g) == 0)).to(dtype).cuda()
            b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t() if nt else torch.randint(-1, 2, (K, N), generator=g).to(dtype).cuda()
            bias = torch.randint(-2, 3, (N,), generator=g).to(dtype).cuda()
            full = torch.randint(-2, 3, (M, N), generator=g).to(dtype).cuda()
            ref = aten_cpu.reference(aten.mm.default, [a.float(), b.float()])
            assert float(ref.abs().max()) <= 192
            ref = ref.to(dtype)
            assert ev.bit_equal(ref, backend[aten.mm.default](a, b).cpu()), (meet, M, N, K, nt)
            out = backend[aten.addmm.default](bias, a, b)
            assert ev.bit_equal((ref.float() + bias.cpu().float()).to(dtype), out.cpu()), (meet, M, N, K, nt, "bias row")
            out = backend[aten.addmm.default](full, a, b, beta=2, alpha=0.5)
            assert ev.bit_equal((0.5 * ref.float() + 2 * full.cpu().float()).to(dtype), out.cpu()), (meet, M, N, K, nt, "full c")
    assert split_seen >= (9 if meet == "inlaunch" else 7), "these shapes are meant to split K"  # (a summing launch pays for fewer of them)
    assert lib.mi355_gemm_status() == 0
    if meet != "inlaunch":
        return
    M, N, K = 1024, 2048, 4096
    a = torch.randint(-1, 2, (M, K), generator=g).to(dtype).cuda()
    a2 = torch.randint(-1, 2, (M, K), generator=g).to(dtype).cuda()
    b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t()
    want, want2 = backend[aten.mm.default](a, b), backend[aten.mm.default](a2, b)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = backend[aten.mm.default](a, b)
        got2 = backend[aten.mm.default](a2, b)
    for rep in range(4):
        got.zero_()
        got2.zero_()
        junk = torch.full((64 << 20,), float(rep), device="cuda")   # eager work that may land on the freed workspace
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert ev.bit_equal(want, got) and ev.bit_equal(want2, got2), ("replay", rep)
        del junk
    assert lib.mi355_gemm_status() == 0


@pytest.mark.parametrize("layout", ["nt", "nn"])
def test_cache_warming_workgroups_change_no_result(backend, layout, gemm_knobs):
    """A launch that leaves CUs without a tile appends workgroups that only read the operands ahead of the tiles
    (warm_operands: the deep-ring 128x128 kernels, the 64x64-tile kernel with its deep ring, the 256x128 form, the
    16x16x32 kernel with one workgroup per tile, with K split inside the launch or not).  With none of them, with
    the planner's count, with a few and with more than there are idle CUs (the count is cut down) every form must
    give the same bits, equal to the oracle on small-integer operands; ragged edges and K ranges included."""
    announce(f"cache-warming workgroups, {layout}")
    g = torch.Generator().manual_seed(53)
    # (M, N, K, forced form or None): tiles x parts stay under 256 so that CUs are left over
    shapes = [(1536, 2048, 4096, None), (1500, 2040, 2112, None), (2048, 768, 3072, None), (1024, 2048, 4096, None),
              (896, 896, 3584, None), (640, 1280, 4096, "64x64"), (4096, 1536, 1536, None), (3072, 2304, 768, None),
              (4000, 1480, 1088, "256x128"), (2304, 4096, 2048, "x16"), (1280, 2560, 1024, "x16"), (1024, 1024, 8192, "ring8"),
              (1024, 1024, 8192, "ring4")]
    for M, N, K, form in shapes:
        dtype = torch.bfloat16 if (M + K) % 512 == 0 else torch.float16
        a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.randint(0, 4, (M, K), generator=g) == 0)).to(dtype).cuda()
        b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t() if layout == "nt" else torch.randint(-1, 2, (K, N), generator=g).to(dtype).cuda()
        bias = torch.randint(-2, 3, (N,), generator=g).to(dtype).cuda()
        ref = aten_cpu.reference(aten.mm.default, [a.float(), b.float()])
        assert float(ref.abs().max()) <= 250
        want = (ref + bias.cpu().float()).to(dtype)
        gemm_knobs.tile(form)
        for count in (None, "0", "5", "32", "250"):
            gemm_knobs.prefetch(count)
            got = backend[aten.addmm.default](bias, a, b)
            torch.cuda.synchronize()
            assert ev.bit_equal(want, got.cpu()), (M, N, K, form, layout, count)
        gemm_knobs.prefetch(None)
        gemm_knobs.tile(None)
    from backendbench_amd import _lib
    assert _lib.load().mi355_gemm_status() == 0


def test_f64_addmm_keeps_alpha_and_beta_in_f64(backend):
    """alpha = 0.1 and beta = 0.3 are not fp32 numbers: an f64 addmm must apply them in f64 (1e-12
    against the oracle, where an fp32 round trip of the scalars leaves 1e-8), and a beta too small for
    fp32 must still count."""
    announce("f64 addmm scalars")
    g = torch.Generator().manual_seed(10)
    c = torch.randn(37, 29, generator=g, dtype=torch.float64)
    a = torch.randn(37, 53, generator=g, dtype=torch.float64)
    b = torch.randn(53, 29, generator=g, dtype=torch.float64)
    got = backend[aten.addmm.default](c.cuda(), a.cuda(), b.cuda(), beta=0.3, alpha=0.1).cpu()
    ref = aten_cpu.reference(aten.addmm.default, [c, a, b], {"beta": 0.3, "alpha": 0.1})
    assert torch.allclose(got, ref, rtol=1e-12, atol=1e-12), (got - ref).abs().max()
    tiny = backend[aten.addmm.default](c.cuda() * 1e60, a.cuda(), b.cuda(), beta=1e-60, alpha=0.0).cpu()
    assert torch.allclose(tiny, c, rtol=1e-12, atol=1e-12)


def test_f64_products_on_the_mfma_kernel(backend):
    """fp64 mm / addmm run on v_mfma_f64_16x16x4_f64 (32x32 tiles for a few dozen tiles, 64x64, 128x128
    from 256 tiles on) for every combination of operand layouts: shapes off the tile and step sizes, K
    down to 1, the three addmm forms.  1e-12 against the oracle, relative to the largest element; integer-valued operands (sums
    below 2^53) must come out exactly."""
    announce("f64 mfma products")
    g = torch.Generator().manual_seed(11)
    shapes = [(1, 1, 1), (3, 5, 7), (16, 4, 16), (17, 33, 65), (65, 17, 63), (129, 1000, 257), (200, 100, 300),
              (2100, 70, 2100), (1000, 40, 1030), (1, 515, 300), (300, 16, 1)]
    for (M, K, N) in shapes:
        for a_t in (False, True):
            for b_t in (False, True):
                a = torch.randn(K, M, generator=g, dtype=torch.float64).t() if a_t else torch.randn(M, K, generator=g, dtype=torch.float64)
                b = torch.randn(N, K, generator=g, dtype=torch.float64).t() if b_t else torch.randn(K, N, generator=g, dtype=torch.float64)
                ref = aten_cpu.reference(aten.mm.default, [a, b])
                got = backend[aten.mm.default](a.cuda(), b.cuda()).cpu()
                assert got.shape == ref.shape
                assert (got - ref).abs().max() <= 1e-12 * max(ref.abs().max().item(), 1.0), (M, K, N, a_t, b_t)
        a = torch.randn(M, K, generator=g, dtype=torch.float64)
        b = torch.randn(K, N, generator=g, dtype=torch.float64)
        for c, kw in ((torch.randn(N, generator=g, dtype=torch.float64), {"beta": 0.3, "alpha": 0.1}),
                      (torch.randn(M, N, generator=g, dtype=torch.float64).t().contiguous().t(), {"beta": -2.0, "alpha": 0.5}),
                      (torch.randn(M, 1, generator=g, dtype=torch.float64), {})):
            ref = aten_cpu.reference(aten.addmm.default, [c, a, b], kw)
            got = backend[aten.addmm.default](c.cuda(), a.cuda(), b.cuda(), **kw).cpu()
            assert (got - ref).abs().max() <= 1e-12 * max(ref.abs().max().item(), 1.0), (M, K, N, kw)
    # integers: every partial sum is exact in fp64, whatever the order of the additions
    ai = torch.randint(-1000, 1000, (300, 700), generator=g).double()
    bi = torch.randint(-1000, 1000, (700, 2100), generator=g).double()
    assert torch.equal(backend[aten.mm.default](ai.cuda(), bi.cuda()).cpu(), aten_cpu.reference(aten.mm.default, [ai, bi]))
    assert torch.equal(backend[aten.mm.default](bi.t().cuda(), ai.t().cuda()).cpu(), aten_cpu.reference(aten.mm.default, [bi.t(), ai.t()]))


@pytest.mark.parametrize("layout", ["nn", "nt"])
@pytest.mark.parametrize("shape", [(200, 330), (1700, 1752), (2100, 2064)])
def test_fp32_gemm_every_k_loop_length(backend, layout, shape):
    """The fp32 MFMA kernel in its three forms: [200, K] x [K, 330] runs on 64x64 tiles (eight-stage
    ring, split along K once K is long enough), [1700, K] x [K, 1752] has 196 tiles of 128x128 (one
    workgroup per CU, eight stages), [2100, K] x [K, 2064] has 289 (four stages, two per CU).  K walks
    through every prologue / steady / drain length of both ring depths; small-integer operands make the
    fp32 accumulation exact in any order, so the sampled rows must be bit-equal to the oracle's."""
    M, N = shape
    announce(f"fp32 GEMM K loop lengths, {layout}, {M}x{N}")
    g = torch.Generator().manual_seed(8)
    rows = torch.unique(torch.cat([torch.randint(0, M, (40,), generator=g), torch.tensor([0, 31, 32, 63, 64, 127, 128, M - 65, M - 64, M - 1])]))
    for K in list(range(16, 16 * 21, 16)) + [400, 1040, 2064]:
        a = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
        if layout[1] == "t":
            b = torch.randint(-2, 3, (N, K), generator=g).float().cuda().t()
        else:
            b = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
        out = backend[aten.mm.default](a, b)
        ref = aten_cpu.reference(aten.mm.default, [a[rows.cuda()], b])
        assert ev.bit_equal(ref, out[rows.cuda()].cpu()), (layout, shape, K)


def test_cpu_tensors_round_trip_through_the_gpu(backend):
    """The smoke suite hands CPU tensors (BackendBench/suite/smoke.py:25,30): the result must
    come back on the CPU and match ATen."""
    announce("smoke suite via directory backend")
    for t in SmokeTestSuite:
        c, p, cr, pr = ev.eval_one_op(t.op, backend[t.op], t.correctness_tests, t.performance_tests)
        assert c == 1.0 and all(r.is_correct for r in cr) and pr[0].successfully_ran
    x = torch.randn(5, 7)
    y = backend[aten.add.Tensor](x, torch.randn(7).cuda())   # mixed devices follow the first tensor
    assert y.device.type == "cpu"
    outs = backend[aten.native_layer_norm.default](x, [7], None, None, 1e-5)
    assert all(o.device.type == "cpu" for o in outs)


def test_out_of_range_index_surfaces_without_an_evaluator(backend, monkeypatch):
    """A caller that never polls (the reference's evaluator, a live model under enable()): the call with
    the bad index returns (its row zero-filled, nothing dereferenced), and once the device has run it the
    next call of any operator of this backend raises IndexError, as a device-side assert of the stock
    kernels would surface at a later call.  After the raise the backend is clean again."""
    from backendbench_amd.ops import check_index_errors

    announce("deferred out-of-range index error")
    monkeypatch.delenv("MI355_SYNC_INDEX_CHECK", raising=False)
    check_index_errors()
    table = torch.randn(11, 6, device="cuda")
    idx = torch.tensor([2, 11, 4], device="cuda")
    got = backend[aten.index_select.default](table, 0, idx)          # does not raise
    torch.cuda.synchronize()
    assert ev.bit_equal(got[0], table[2]) and ev.bit_equal(got[2], table[4])
    assert torch.count_nonzero(got[1]).item() == 0                       # the bad row is zero-filled
    with pytest.raises(IndexError, match="earlier index_select / embedding / gather"):
        backend[aten.relu.default](table)                                # any later call reports it
    assert ev.bit_equal(backend[aten.relu.default](table).cpu(), torch.relu(table).cpu())   # clean again
    got = backend[aten.gather.default](table, 1, torch.tensor([[7]], device="cuda"))
    torch.cuda.synchronize()
    with pytest.raises(IndexError):
        backend[aten.embedding.default](table, torch.tensor([1], device="cuda"))
    good = backend[aten.embedding.default](table, torch.tensor([1], device="cuda"))
    torch.cuda.synchronize()
    backend[aten.relu.default](table)                                    # nothing pending: no raise
    assert ev.bit_equal(good, table[1:2])
    check_index_errors()


def test_error_behaviour_matches_the_oracle(backend, monkeypatch):
    announce("error behaviour")
    monkeypatch.setenv("MI355_SYNC_INDEX_CHECK", "1")
    table = torch.randn(11, 6, device="cuda")
    for bad in ([11], [-1]):
        idx = torch.tensor(bad, device="cuda")
        assert aten_cpu.raises(aten.index_select.default, [table, 0, idx]) is IndexError
        with pytest.raises(IndexError):
            backend[aten.index_select.default](table, 0, idx)
        with pytest.raises(IndexError):
            backend[aten.embedding.default](table, idx)
    with pytest.raises(IndexError):   # selecting along the last dim goes through the LDS-staged kernel
        backend[aten.index_select.default](table, 1, torch.tensor([0, 6, 2], device="cuda"))
    with pytest.raises((RuntimeError, IndexError)):
        backend[aten.gather.default](table, 1, torch.tensor([[-1]], device="cuda"))
    # a good call after a bad one is clean again
    assert ev.bit_equal(backend[aten.index_select.default](table, 0, torch.tensor([3], device="cuda")), table[3:4])
    ints = torch.arange(12, device="cuda").reshape(3, 4)
    for op, args in ((aten.mean.dim, [ints, [-1]]), (aten.amax.default, [torch.zeros(4, 0, device="cuda"), [-1]]),
                     (aten.argmax.default, [torch.zeros(4, 0, device="cuda"), -1]),
                     (aten.mm.default, [torch.zeros(2, 3, device="cuda"), torch.zeros(4, 5, device="cuda")]),
                     (aten.clamp.default, [torch.zeros(2, device="cuda")]),
                     (aten.sum.dim_IntList, [torch.zeros(2, 3, device="cuda"), [2]]),
                     (aten._softmax.default, [torch.zeros(2, 3, device="cuda"), 5, False])):
        expected = aten_cpu.raises(op, args)
        assert expected is not None, op
        with pytest.raises(expected):
            backend[op](*args)


def test_live_dispatcher_override_runs_our_kernels(backend):
    """enable(dispatch_key="CUDA") routes torch calls on HIP tensors to the directory backend
    (BackendBench/__init__.py:70-143).  A small transformer-style block must give the same
    answer with and without the override, and must not recurse."""
    import backendbench_amd
    from backendbench_amd import _lib

    announce("enable() with real kernels")
    g = torch.Generator().manual_seed(0)
    V, D, H, T = 1000, 256, 512, 64
    emb = (torch.randn(V, D, generator=g) * 0.02).bfloat16().cuda()
    w1 = (torch.randn(D, H, generator=g) * 0.05).bfloat16().cuda()
    b1 = (torch.randn(H, generator=g) * 0.05).bfloat16().cuda()
    w2 = (torch.randn(H, D, generator=g) * 0.05).bfloat16().cuda()
    gamma, beta = torch.ones(D).bfloat16().cuda(), torch.zeros(D).bfloat16().cuda()
    tok = torch.randint(0, V, (T,), generator=g).cuda()

    def block():
        x = torch.nn.functional.embedding(tok, emb)
        x = torch.nn.functional.layer_norm(x, (D,), gamma, beta, 1e-5)
        h = torch.relu(torch.addmm(b1, x, w1))
        y = torch.mm(h, w2) + x
        p = torch.softmax(y.float(), dim=-1)
        return p, p.argmax(-1), y.sum(-1), y.amax(-1)

    plain = block()
    calls = []
    lib = _lib.load()
    real = lib.mi355_gemm

    with backendbench_amd.BackendBench.enable(kernel_dir=os.path.join(ROOT, "generated_kernels"), dispatch_key="CUDA"):
        from backendbench_amd.ops import _common

        orig = _common.launch
        _common_launch_names = calls

        def spy(name, *a):
            _common_launch_names.append(name)
            return orig(name, *a)

        import backendbench_amd.ops.elementwise as e, backendbench_amd.ops.reduce as r, backendbench_amd.ops.matmul as m, backendbench_amd.ops.index as i
        mods = (e, r, m, i)
        for mod in mods:
            mod.launch = spy
        try:
            ours = block()
            torch.cuda.synchronize()
        finally:
            for mod in mods:
                mod.launch = orig
    assert real is lib.mi355_gemm
    for name in ("mi355_index_select", "mi355_layer_norm", "mi355_gemm", "mi355_unary", "mi355_binary",
                 "mi355_softmax", "mi355_reduce"):
        assert name in calls, f"{name} was not reached through the dispatcher: {sorted(set(calls))}"
    assert torch.equal(plain[1].cpu(), ours[1].cpu())
    for a, b in zip(plain, ours):
        assert ev.allclose(a.cpu(), b.cpu())
    again = block()  # override gone
    assert ev.allclose(plain[0].cpu(), again[0].cpu())


def test_hip_graph_replays_match_eager(backend):
    """The kernels are launched on torch's current stream, so a HIP graph captures them.  Every
    replay (with eager work and synchronisations in between) must reproduce the eager result."""
    announce("hip graph capture/replay")
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(512, 4096, generator=g) * 2).bfloat16().cuda()
    w = (torch.randn(4096, 512, generator=g) * 0.02).bfloat16().cuda()
    gamma, beta = torch.ones(4096).bfloat16().cuda(), torch.zeros(4096).bfloat16().cuda()
    idx = torch.randint(0, 512, (300,), generator=g).cuda()

    def work(inp):
        y, mean, rstd = backend[aten.native_layer_norm.default](inp, [4096], gamma, beta, 1e-5)
        p = backend[aten._softmax.default](y, -1, False)
        h = backend[aten.mm.default](p, w)
        s = backend[aten.sum.dim_IntList](h, [-1])
        e = backend[aten.embedding.default](inp, idx)
        a = backend[aten.argmax.default](h.float(), -1)
        return y, p, h, s, e, a, mean

    eager = [t.clone() for t in work(x)]   # also the warm-up: library load, LDS attribute, error flag
    torch.cuda.synchronize()
    static_in = x.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = work(static_in)
    for rep in range(4):
        static_in.copy_(x if rep % 2 == 0 else x.flip(0))
        graph.replay()
        torch.cuda.synchronize()
        want = eager if rep % 2 == 0 else [t.clone() for t in work(x.flip(0))]
        torch.cuda.synchronize()
        for o, e_ in zip(outs, want):
            assert ev.allclose(e_.cpu(), o.cpu(), exact=not o.dtype.is_floating_point), f"replay {rep} differs"


def _t(shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _inplace_cases():
    f32, bf16, f16, i32 = torch.float32, torch.bfloat16, torch.float16, torch.int32
    return [
        ("add_.same", aten.add_.Tensor, lambda: ([_t((33, 65)), _t((33, 65), seed=1)], {})),
        ("add_.alpha_bcast", aten.add_.Tensor, lambda: ([_t((33, 65), bf16), _t((65,), bf16, seed=1)], {"alpha": -0.5})),
        ("add_.mixed_dtype", aten.add_.Tensor, lambda: ([_t((17, 40), bf16), _t((17, 40), f32, seed=1)], {})),
        ("add_.transposed_self", aten.add_.Tensor, lambda: ([_t((40, 24), f16).t(), _t((24, 40), f16, seed=1)], {})),
        ("add_.int", aten.add_.Tensor, lambda: ([torch.arange(60, dtype=i32).reshape(6, 10), torch.arange(10, dtype=i32)], {"alpha": 3})),
        ("add_.zero_d_other", aten.add_.Tensor, lambda: ([_t((9, 9)), torch.tensor(2.5)], {})),
        ("add_.empty", aten.add_.Tensor, lambda: ([torch.empty(0, 8), torch.empty(0, 8)], {})),
        ("mul_.same", aten.mul_.Tensor, lambda: ([_t((128, 130), bf16), _t((128, 130), bf16, seed=1)], {})),
        ("mul_.bcast_col", aten.mul_.Tensor, lambda: ([_t((31, 70)), _t((31, 1), seed=1)], {})),
        ("mul_.sliced_self", aten.mul_.Tensor, lambda: ([_t((20, 64))[:, 3:35], _t((20, 32), seed=1)], {})),
        ("relu_.f16", aten.relu_.default, lambda: ([_t((1000,), f16)], {})),
        ("relu_.transposed", aten.relu_.default, lambda: ([_t((12, 50)).t()], {})),
        ("relu_.int", aten.relu_.default, lambda: ([torch.arange(-20, 20, dtype=i32)], {})),
        ("clamp_.both", aten.clamp_.default, lambda: ([_t((33, 65)), -0.25, 0.5], {})),
        ("clamp_.min_only", aten.clamp_.default, lambda: ([_t((33, 65), bf16), 0.0], {})),
        ("clamp_.max_kw", aten.clamp_.default, lambda: ([_t((7, 5, 3), f16)], {"max": 0.1})),
        ("add_.Scalar", aten.add_.Scalar, lambda: ([_t((33, 65), bf16), 1.5], {"alpha": 2})),
        ("mul_.Scalar", aten.mul_.Scalar, lambda: ([_t((33, 65)), 0.125], {})),
        ("mul_.Scalar_int", aten.mul_.Scalar, lambda: ([torch.arange(60, dtype=i32).reshape(6, 10), 3], {})),
        ("clamp_min_", aten.clamp_min_.default, lambda: ([_t((33, 65)), 0.1], {})),
        ("clamp_max_", aten.clamp_max_.default, lambda: ([_t((7, 5), f16), -0.2], {})),
        ("clamp_.Tensor", aten.clamp_.Tensor, lambda: ([_t((33, 65)), _t((65,), seed=1) - 1, _t((65,), seed=2) + 1], {})),
        ("clamp_.Tensor_transposed_self", aten.clamp_.Tensor, lambda: ([_t((24, 40)).t(), _t((40, 24), seed=1) - 1], {})),
        ("addmm_", aten.addmm_.default, lambda: ([_t((64, 32)), _t((64, 96), seed=1), _t((96, 32), seed=2)], {"beta": 0.5, "alpha": 2.0})),
    ]


@pytest.mark.parametrize("case", _inplace_cases(), ids=[c[0] for c in _inplace_cases()])
def test_inplace_overloads_write_through_self(backend, case):
    """add_/mul_/relu_/clamp_ return `self` itself, leave its layout alone, and hold the values
    ATen's in-place overload leaves in a CPU clone of the same inputs."""
    key, op, make = case
    announce(key)
    args, kwargs = make()
    args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    base = args[0]
    cpu_args = [a.cpu().clone() if isinstance(a, torch.Tensor) else a for a in args]
    if not base.is_contiguous():   # clone() would densify: rebuild the same view on the CPU
        cpu_args[0] = torch.empty_strided(base.shape, base.stride(), dtype=base.dtype).copy_(base.cpu())
    ptr, stride = base.data_ptr(), base.stride()
    res = backend[op](*args, **kwargs)
    torch.cuda.synchronize()
    ref = op(*cpu_args, **kwargs)
    assert res is base and res.data_ptr() == ptr and res.stride() == stride
    assert ev.allclose(ref, res.cpu(), exact=not ref.dtype.is_floating_point), key


def test_inplace_overloads_reject_what_aten_rejects(backend):
    announce("in-place error behaviour")
    ints = torch.arange(6, device="cuda")
    for op, args in ((aten.add_.Tensor, [ints, torch.ones(6, device="cuda")]),          # float result into int self
                     (aten.mul_.Tensor, [torch.ones(6, device="cuda"), torch.ones(2, 6, device="cuda")]),  # self would grow
                     (aten.clamp_.default, [torch.ones(3, device="cuda")])):
        cpu_args = [a.cpu().clone() if isinstance(a, torch.Tensor) else a for a in args]
        expected = aten_cpu.raises(op, cpu_args)
        assert expected is not None, op
        with pytest.raises(expected):
            backend[op](*args)
    assert torch.equal(ints.cpu(), torch.arange(6))   # nothing was written
    # memory overlap between the written-to tensor and an operand, or inside the written-to tensor
    def overlap_cases(dev):
        sq = torch.arange(9.0, device=dev).reshape(3, 3)
        return [(aten.add_.Tensor, lambda: [sq.clone(), None], "t"), (aten.add_.Tensor, lambda: [sq.clone(), None], "row"),
                (aten.mul_.Tensor, lambda: [torch.ones(3, device=dev).expand(2, 3), torch.ones(2, 3, device=dev)], None),
                (aten.relu_.default, lambda: [torch.ones(3, device=dev).expand(2, 3)], None),
                (aten.clamp_.default, lambda: [torch.ones(3, device=dev).expand(2, 3), 0.0, 0.5], None)]
    for (op, mk, view), (_, mk_cpu, _v) in zip(overlap_cases("cuda"), overlap_cases("cpu")):
        def fill(args):
            if view == "t": args[1] = args[0].t()
            if view == "row": args[1] = args[0][0]
            return args
        expected = aten_cpu.raises(op, fill(mk_cpu()))
        assert expected is RuntimeError, (op, view)
        with pytest.raises(RuntimeError, match="single memory location"):
            backend[op](*fill(mk()))
    x = torch.arange(9.0, device="cuda").reshape(3, 3)
    assert ev.bit_equal(backend[aten.add_.Tensor](x, x).cpu(), torch.arange(9.0).reshape(3, 3) * 2)   # full overlap is fine
    # integer clamp bounds the dtype cannot hold (a negative bound on uint8 wraps, as in ATen)
    for dtype, kw in ((torch.int8, {"max": 300}), (torch.uint8, {"min": -5}), (torch.uint8, {"min": -300}), (torch.int16, {"min": -40000}),
                      (torch.uint8, {"max": 256})):
        t = torch.arange(0, 100, 7).to(dtype)
        expected = aten_cpu.raises(aten.clamp.default, [t], kw)
        if expected is None:
            assert ev.bit_equal(aten.clamp.default(t, **kw), backend[aten.clamp.default](t.cuda(), **kw).cpu()), (dtype, kw)
        else:
            with pytest.raises(expected, match="without overflow"):
                backend[aten.clamp.default](t.cuda(), **kw)


def _out_cases():
    f32, bf16, i64 = torch.float32, torch.bfloat16, torch.int64
    idx = torch.tensor([4, 0, 4, 2])
    gidx = torch.randint(0, 9, (9, 5), generator=torch.Generator().manual_seed(5))
    cond = _t((6, 30), seed=9) > 0
    return [
        ("add.out", aten.add.out, [_t((6, 30)), _t((30,), seed=1)], {"alpha": 2}, ((6, 30), f32)),
        ("add.out_cast", aten.add.out, [_t((6, 30)), _t((6, 30), seed=1)], {}, ((6, 30), bf16)),
        ("add.out_resized", aten.add.out, [_t((6, 30)), _t((6, 30), seed=1)], {}, ((0,), f32)),
        ("mul.out", aten.mul.out, [_t((6, 30), bf16), _t((6, 30), bf16, seed=1)], {}, ((6, 30), bf16)),
        ("maximum.out", aten.maximum.out, [_t((6, 30)), _t((6, 30), seed=1)], {}, ((6, 30), f32)),
        ("relu.out", aten.relu.out, [_t((6, 30))], {}, ((6, 30), f32)),
        ("clamp.out", aten.clamp.out, [_t((6, 30)), -0.1, 0.3], {}, ((6, 30), f32)),
        ("where.self_out", aten.where.self_out, [cond, _t((6, 30)), _t((6, 30), seed=1)], {}, ((6, 30), f32)),
        ("sum.IntList_out", aten.sum.IntList_out, [_t((6, 30, 4)), [1]], {"keepdim": True}, ((6, 1, 4), f32)),
        ("sum.IntList_out_dtype", aten.sum.IntList_out, [_t((6, 30), bf16), [-1]], {"dtype": f32}, ((6,), f32)),
        ("mean.out", aten.mean.out, [_t((6, 30)), [0]], {}, ((30,), f32)),
        ("amax.out", aten.amax.out, [_t((6, 30)), [-1]], {}, ((6,), f32)),
        ("argmax.out", aten.argmax.out, [_t((6, 30)), 1], {}, ((6,), i64)),
        ("_softmax.out", aten._softmax.out, [_t((6, 30)), -1, False], {}, ((6, 30), f32)),
        ("mm.out", aten.mm.out, [_t((64, 96), bf16), _t((96, 32), bf16, seed=1)], {}, ((64, 32), bf16)),
        ("addmm.out", aten.addmm.out, [_t((32,)), _t((64, 96)), _t((96, 32), seed=1)], {"beta": 0.5, "alpha": 2.0}, ((64, 32), f32)),
        ("index_select.out", aten.index_select.out, [_t((9, 5)), 0, idx], {}, ((4, 5), f32)),
        ("gather.out", aten.gather.out, [_t((9, 5)), 0, gidx], {}, ((9, 5), f32)),
        ("add.Scalar_out", aten.add.Scalar_out, [_t((6, 30)), 2.5], {"alpha": 2}, ((6, 30), f32)),
        ("mul.Scalar_out", aten.mul.Scalar_out, [_t((6, 30), bf16), 3], {}, ((6, 30), bf16)),
        ("minimum.out", aten.minimum.out, [_t((6, 30)), _t((30,), seed=1)], {}, ((6, 30), f32)),
        ("clamp.Tensor_out", aten.clamp.Tensor_out, [_t((6, 30)), _t((30,), seed=1) - 1, _t((30,), seed=2) + 1], {}, ((6, 30), f32)),
        ("clamp_min.out", aten.clamp_min.out, [_t((6, 30)), 0.1], {}, ((6, 30), f32)),
        ("clamp_max.out", aten.clamp_max.out, [_t((6, 30), bf16), -0.1], {}, ((3,), bf16)),
        ("_log_softmax.out", aten._log_softmax.out, [_t((6, 30)), -1, False], {}, ((6, 30), f32)),
        ("sum.out", aten.sum.out, [_t((6, 30))], {}, ((), f32)),
        ("mean.dtype_out", aten.mean.dtype_out, [_t((6, 30), bf16)], {"dtype": f32}, ((), f32)),
        ("embedding.out", aten.embedding.out, [_t((9, 5)), idx], {}, ((4, 5), f32)),
    ]


@pytest.mark.parametrize("case", _out_cases(), ids=[c[0] for c in _out_cases()])
def test_out_overloads_fill_the_given_tensor(backend, case):
    """`<op>.out(..., out=t)` returns `t` itself holding what ATen's out= overload writes on the
    CPU, including the cast into `t`'s dtype and the resize of a wrongly shaped `t`."""
    import warnings

    key, op, args, kwargs, (oshape, odtype) = case
    announce(key)
    out = torch.full(oshape, 7, dtype=odtype).cuda()
    gpu_args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    res = backend[op](*gpu_args, out=out, **kwargs)
    torch.cuda.synchronize()
    from backendbench_amd.ops import check_index_errors

    check_index_errors()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        ref = op(*args, out=torch.full(oshape, 7, dtype=odtype), **kwargs)
    assert res is out
    assert ev.allclose(ref, res.cpu(), exact=not ref.dtype.is_floating_point or key in ("where.self_out", "index_select.out", "gather.out", "embedding.out")), key


@pytest.mark.parametrize("shape,dtype", [((2, 786432), torch.float32), ((3, 100001), torch.float32), ((1, 1 << 20), torch.bfloat16),
                                         ((5, 65536), torch.float16), ((2, 70000), torch.float64), ((63, 32768), torch.bfloat16)])
def test_few_very_long_rows_split_over_the_chip(backend, shape, dtype):
    """A handful of rows of tens of thousands of elements: softmax, log-softmax and layer norm cut every row
    into chunks (two launches, partial states in a scratch buffer).  Aligned and odd row lengths, every
    float dtype, a +inf and a NaN planted in different rows; compared with the oracle to the usual bar."""
    from backendbench_amd import _lib
    announce(f"few long rows {shape} {dtype}")
    rows, n = shape
    assert _lib.load().mi355_row_workspace_bytes(rows, n, _lib.dtype_code(dtype)) > 0, "meant to take the split form"
    g = torch.Generator().manual_seed(rows * 7 + n)
    x = (torch.randn(shape, generator=g) * 3).to(dtype)
    x[0, n // 3] = 40.0                                   # one dominant element
    if rows > 2:
        x[1, 5] = float("inf")
        x[2, n - 1] = float("nan")
    xg = x.cuda()
    for op, args in ((aten._softmax.default, [xg, -1, False]), (aten._log_softmax.default, [xg, 1, False])):
        got = backend[op](*args)
        ref = aten_cpu.reference(op, args)
        assert ev.allclose(ref, got.cpu()), (op, ev.compute_errors(ref, got.cpu()))
    if dtype in (torch.float16, torch.bfloat16):
        got = backend[aten._softmax.default](xg, -1, True)
        assert got.dtype == torch.float32 and ev.allclose(aten_cpu.reference(aten._softmax.default, [xg, -1, True]), got.cpu())
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype).cuda()
    b = (0.1 * torch.randn(n, generator=g)).to(dtype).cuda()
    finite = torch.nan_to_num(x, nan=0.5, posinf=2.0).cuda()
    for params in ((w, b), (None, None), (w, None)):
        args = [finite, [n], params[0], params[1], 1e-5]
        got = backend[aten.native_layer_norm.default](*args)
        ref = aten_cpu.reference(aten.native_layer_norm.default, args)
        for r, o in zip(ref, got):
            assert r.shape == o.shape and r.dtype == o.dtype and ev.allclose(r, o.cpu()), ev.compute_errors(r, o.cpu())
    if dtype == torch.bfloat16:   # fp32 gamma / beta on a half input
        args = [finite, [n], w.float(), b.float(), 1e-5]
        got = backend[aten.native_layer_norm.default](*args)
        ref = aten_cpu.reference(aten.native_layer_norm.default, args)
        assert all(ev.allclose(r, o.cpu()) for r, o in zip(ref, got))


def test_native_layer_norm_out_fills_three_tensors(backend):
    """native_layer_norm.out (BackendBench/scripts/op_map.py:776): y, mean and rstd go into out0 / out1 / out2,
    which are resized when their shapes differ, and the same three objects come back."""
    announce("native_layer_norm.out")
    x, w, b = _t((6, 5, 40), seed=3), _t((40,), seed=4), _t((40,), seed=5)
    outs = [torch.full((1,), 7.0).cuda(), torch.full((6, 5, 1), 7.0).cuda(), torch.empty(0).cuda()]
    res = backend[aten.native_layer_norm.out](x.cuda(), [40], w.cuda(), b.cuda(), 1e-5, out0=outs[0], out1=outs[1], out2=outs[2])
    torch.cuda.synchronize()
    ref = aten.native_layer_norm.out(x, [40], w, b, 1e-5, out0=torch.empty(0), out1=torch.empty(0), out2=torch.empty(0))
    assert len(res) == 3 and all(r is o for r, o in zip(res, outs))
    for r, want in zip(res, ref):
        assert r.shape == want.shape and ev.allclose(want, r.cpu())


def test_out_overload_rejects_a_narrowing_cast(backend):
    announce("out= error behaviour")
    a = torch.ones(4, device="cuda")
    out = torch.zeros(4, dtype=torch.int32, device="cuda")
    assert aten_cpu.raises(aten.add.out, [a.cpu(), a.cpu()], {"out": out.cpu()}) is RuntimeError
    with pytest.raises(RuntimeError):
        backend[aten.add.out](a, a, out=out)


def test_variant_overloads_through_the_live_dispatcher(backend):
    """Python's in-place operators, out= keywords and the sibling overloads reach the variant
    slots under enable(), with results equal to the stock run."""
    import backendbench_amd
    import backendbench_amd.ops.elementwise as e
    import backendbench_amd.ops.reduce as r
    from backendbench_amd.ops import _common

    announce("enable(): in-place / out= / sibling overloads")
    x0 = _t((48, 200), torch.bfloat16, seed=1).cuda()
    y0 = _t((48, 200), torch.bfloat16, seed=2).cuda()
    lo = _t((200,), torch.bfloat16, seed=3, scale=0.1).cuda() - 0.5

    def work():
        x = x0.clone()
        x += y0
        x *= 0.5
        x.mul_(y0)
        z = torch.empty_like(x)
        torch.add(x, y0, alpha=2, out=z)
        z.relu_()
        z.clamp_(max=1.5)
        c = torch.clamp(x, min=lo)
        m = torch.minimum(c, y0)
        lp = torch.log_softmax(m.float(), dim=-1)
        cm = torch.clamp_min(x, -0.25).clamp_max(0.75)
        return x, z, c, m, lp, cm

    plain = work()
    calls = []
    orig = _common.launch

    def spy(name, *a):
        calls.append((name, a[0] if name in ("mi355_binary", "mi355_unary") else None))
        return orig(name, *a)

    with backendbench_amd.BackendBench.enable(kernel_dir=os.path.join(ROOT, "generated_kernels"), dispatch_key="CUDA"):
        e.launch = r.launch = spy
        try:
            ours = work()
            torch.cuda.synchronize()
        finally:
            e.launch = r.launch = orig
    from backendbench_amd import _lib

    names = [n for n, _ in calls]
    assert names.count("mi355_binary") >= 6 and names.count("mi355_unary") >= 4 and "mi355_softmax" in names
    assert ("mi355_binary", _lib.MINIMUM) in calls and ("mi355_binary", _lib.MAXIMUM) in calls
    for a, b in zip(plain, ours):
        assert a.dtype == b.dtype and ev.allclose(a.cpu(), b.cpu())


def test_trace_replay_scores_every_op_correct(backend):
    """A text trace in the reference's TorchBench format (BackendBench/data_loaders.py:43-91,
    suite/torchbench.py:39-105) with transformer-shaped inputs, replayed through
    eval_one_op as the reference's `--suite torchbench` does: tensors are drawn on the GPU,
    the reference value is the stock ATen kernel on the same tensors (eval.py:100), every
    operator must score 1.0."""
    from backendbench_amd.suite.trace import TraceTestSuite

    suite = TraceTestSuite("trace", os.path.join(ROOT, "tests", "golden", "transformer_block_trace.txt"), topn=None)
    seen = 0
    for t in suite:
        announce(f"trace {t.op.__name__}")
        torch.manual_seed(seen)
        c, p, cr, pr = ev.eval_one_op(t.op, backend[t.op], t.correctness_tests, t.performance_tests)
        bad = [r for r in cr if not r.is_correct]
        assert c == 1.0, f"{t.op.__name__}: {[(r.args, r.error_msg, r.max_abs_error) for r in bad]}"
        assert all(r.successfully_ran for r in pr), [r.error_msg for r in pr if not r.successfully_ran]
        print(f"[trace] {t.op.__name__:32s} speedup over the stock GPU kernel {p:6.2f}x  "
              + " ".join(f"{r.speedup:.2f}" for r in pr), flush=True)
        seen += 1
    assert seen == 20


def test_evaluator_scores_the_whole_gpu_suite(backend):
    """The evaluator's own flow (reference from the stock operator on the same device, then the
    directory backend) over every operator of the GPU-built suite: all correct, a finite speed-up
    for every operator.  Cases that ATen's GPU kernels refuse stay out of a suite built for the GPU."""
    import math

    from backendbench_amd.suite import BaselineTestSuite

    announce("evaluator over the GPU baseline suite")
    suite = BaselineTestSuite("cuda", scale=0.05)
    n_ops = 0
    for test in suite:
        assert test.op in backend, test.op
        c_score, p_score, c_res, p_res = ev.eval_one_op(test.op, backend[test.op], test.correctness_tests,
                                                        test.performance_tests)
        wrong = [r.args[:120] for r in c_res if not r.is_correct]
        assert c_score == 1.0 and not wrong, (test.op, wrong[:3])
        assert math.isfinite(float(p_score)) and float(p_score) > 0, test.op
        n_ops += 1
    assert n_ops == 28 + 26   # functional overloads + one timed (and one checked) case per out= overload
    assert not any(c.extra.get("cpu_reference_only") for t in suite for c in [x.case for x in t.correctness_tests])


def test_tensors_beyond_2_to_31_elements(backend):
    """Element counts and byte offsets past 2^31 / 2^32: the kernels index with 64 bits."""
    announce("tensors beyond 2^31 elements")
    n = (1 << 31) + 4096 + 3
    g = torch.Generator().manual_seed(11)
    x = torch.randint(-100, 100, (n,), generator=g, dtype=torch.int8)
    xg = x.cuda()
    y = backend[aten.relu.default](xg)
    torch.cuda.synchronize()
    assert torch.equal(y[-(1 << 20):].cpu(), torch.relu(x[-(1 << 20):])) and torch.equal(y[: 1 << 20].cpu(), torch.relu(x[: 1 << 20]))
    mid = (1 << 31) - 512
    assert torch.equal(y[mid: mid + 1024].cpu(), torch.relu(x[mid: mid + 1024]))
    s = backend[aten.sum.default](xg)
    assert s.dtype == torch.int64 and int(s.item()) == int(x.sum(dtype=torch.int64).item())
    del y, xg
    # rows whose byte offset exceeds 2^32
    table = torch.empty(70000, 16384, dtype=torch.float32, device="cuda")
    rows = torch.tensor([69999, 0, 65537, 33000, 69998], device="cuda")
    table[rows] = torch.arange(5, dtype=torch.float32, device="cuda")[:, None] + 1
    out = backend[aten.index_select.default](table, 0, rows)
    emb = backend[aten.embedding.default](table, rows.view(5, 1))
    torch.cuda.synchronize()
    want = (torch.arange(5, dtype=torch.float32)[:, None] + 1).expand(5, 16384)
    assert torch.equal(out.cpu(), want) and torch.equal(emb.cpu().view(5, 16384), want)


def test_row_kernels_beyond_2_to_31_elements(backend):
    """Row-wise kernels and the GEMM on one 4 GiB f16 buffer viewed as rows: the first and the last rows
    (element offsets past 2^31) are compared with the CPU on the same slices."""
    announce("row kernels beyond 2^31 elements")
    n = (1 << 31) + 2048
    a = torch.empty(n, dtype=torch.float16, device="cuda")
    a.normal_(generator=torch.Generator(device="cuda").manual_seed(5))
    a[n - 7] = 100.0
    assert int(backend[aten.argmax.default](a).item()) == n - 7

    def ends(t, k):
        return torch.cat([t[:k], t[-k:]]).cpu()

    def close(got, want):
        return torch.allclose(got.float(), want.float(), atol=1e-2, rtol=1e-2)

    a8 = a.view(-1, 8)
    got = backend[aten.amax.default](a8, [1])
    assert torch.equal(ends(got, 4096), ends(a8, 4096).amax(1))
    got = backend[aten._softmax.default](a8, -1, False)
    assert close(ends(got, 4096), torch.softmax(ends(a8, 4096).float(), -1))
    del got
    a1k = a.view(-1, 1024)
    y, mean, rstd = backend[aten.native_layer_norm.default](a1k, [1024], None, None, 1e-5)
    wy, wm, wr = torch.native_layer_norm(ends(a1k, 512).float(), [1024], None, None, 1e-5)
    assert close(ends(y, 512), wy) and close(ends(mean, 512), wm) and close(ends(rstd, 512), wr)
    del y
    w = torch.randn(1024, 64, generator=torch.Generator().manual_seed(6)).to(torch.float16)
    got = backend[aten.mm.default](a1k, w.cuda())
    want = ends(a1k, 512).float() @ w.float()
    assert torch.allclose(ends(got, 512).float(), want, atol=0.25, rtol=1e-2)  # |sum of 1024 products| ~ 32, f16 output
    del got
    a512 = a.view(-1, 512)
    idx = torch.randint(0, a512.shape[0], (3000, 512), generator=torch.Generator().manual_seed(7))
    idx[-1] = a512.shape[0] - 1
    got = backend[aten.gather.default](a512, 0, idx.cuda())
    sample = torch.tensor([0, 1500, 2999])
    want = torch.gather(a.cpu().view(-1, 512), 0, idx[sample])
    assert torch.equal(got[sample.cuda()].cpu(), want)


@pytest.mark.parametrize("n", [2049, 197, 50257, 8193])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_misaligned_rows_see_exactly_their_own_elements(backend, n, dtype):
    """Odd row lengths put rows off 16-byte boundaries; the row kernels then read the aligned
    window around each row.  Markers on the first and last element of alternating rows make
    any element dropped at a row's ends, or leaked in from a neighbouring row, change the result."""
    announce(f"row boundaries n={n} {dtype}")
    rows = 64 if n > 20000 else 300
    g = torch.Generator().manual_seed(n)
    x = -torch.rand(rows, n, generator=g)            # everything in (-1, 0]
    x[0::2, -1] = 500.0                               # even rows: the maximum is the last element
    x[1::4, 0] = 900.0                                # some odd rows: the maximum is the first element
    x = x.to(dtype)
    xg = x.cuda()
    for op, args in ((aten.amax.default, [[-1]]), (aten.argmax.default, [-1]), (aten.sum.dim_IntList, [[-1]]),
                     (aten._softmax.default, [-1, False]), (aten._log_softmax.default, [-1, False])):
        got = backend[op](xg, *args)
        torch.cuda.synchronize()
        ref = aten_cpu.reference(op, [x, *args])
        assert ev.allclose(ref, got.cpu(), exact=op is aten.argmax.default), f"{op.__name__} n={n}"
    w = torch.rand(n, generator=g).to(dtype)
    got = backend[aten.native_layer_norm.default](xg, [n], w.cuda(), None, 1e-5)
    ref = aten_cpu.reference(aten.native_layer_norm.default, [x, [n], w, None, 1e-5])
    assert ev.allclose(ref, tuple(t.cpu() for t in got)), f"layer_norm n={n}"
    bias = torch.rand(n, generator=g).to(dtype)
    got = backend[aten.native_layer_norm.default](xg, [n], w.cuda(), bias.cuda(), 1e-5)
    ref = aten_cpu.reference(aten.native_layer_norm.default, [x, [n], w, bias, 1e-5])
    assert ev.allclose(ref, tuple(t.cpu() for t in got)), f"layer_norm with bias n={n}"
    # the same through a view that starts one element into its storage
    flat = torch.cat([torch.zeros(1, dtype=dtype), x.reshape(-1)]).cuda()
    view = flat[1:].view(rows, n)
    assert view.data_ptr() % 16 != 0
    assert ev.allclose(aten_cpu.reference(aten.amax.default, [x, [-1]]), backend[aten.amax.default](view, [-1]).cpu())
    assert ev.allclose(aten_cpu.reference(aten._softmax.default, [x, -1, False]), backend[aten._softmax.default](view, -1, False).cpu())
    got = backend[aten.native_layer_norm.default](view, [n], None, None, 1e-5)
    ref = aten_cpu.reference(aten.native_layer_norm.default, [x, [n], None, None, 1e-5])
    assert ev.allclose(ref, tuple(t.cpu() for t in got)), f"layer_norm on an offset view n={n}"


@pytest.mark.parametrize("family", ["gpt2", "bert"])
def test_transformers_model_under_the_dispatcher_override(backend, family):
    """A randomly initialised Hugging Face model (built from a config, nothing downloaded) gives
    the same hidden states with the 68 slots overriding ATen's HIP kernels as without, in fp32
    and in bf16; the spy shows the model really runs through the C ABI."""
    transformers = pytest.importorskip("transformers")
    import backendbench_amd
    from backendbench_amd.ops import _common

    announce(f"transformers {family} under enable()")
    torch.manual_seed(0)
    if family == "gpt2":
        cfg = transformers.GPT2Config(n_layer=2, n_head=4, n_embd=256, n_positions=128, vocab_size=1003,
                                      resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
        model = transformers.GPT2LMHeadModel(cfg)
    else:
        cfg = transformers.BertConfig(num_hidden_layers=2, num_attention_heads=4, hidden_size=256, intermediate_size=1024,
                                      vocab_size=1003, max_position_embeddings=128, hidden_dropout_prob=0.0,
                                      attention_probs_dropout_prob=0.0)
        model = transformers.BertModel(cfg)
    cfg._attn_implementation = "eager"
    ids = torch.randint(0, 1003, (4, 96), generator=torch.Generator().manual_seed(1)).cuda()
    for dtype in (torch.float32, torch.bfloat16):
        m = model.to(device="cuda", dtype=dtype).eval()
        with torch.no_grad():
            plain = m(ids)[0]
        calls = []
        orig = _common.launch
        import backendbench_amd.ops.elementwise as e, backendbench_amd.ops.reduce as r, backendbench_amd.ops.matmul as mm_, backendbench_amd.ops.index as ix

        def spy(name, *a):
            calls.append(name)
            return orig(name, *a)

        with backendbench_amd.BackendBench.enable(kernel_dir=os.path.join(ROOT, "generated_kernels"), dispatch_key="CUDA"):
            for mod in (e, r, mm_, ix):
                mod.launch = spy
            try:
                with torch.no_grad():
                    ours = m(ids)[0]
                torch.cuda.synchronize()
            finally:
                for mod in (e, r, mm_, ix):
                    mod.launch = orig
        from backendbench_amd.ops import check_index_errors

        check_index_errors()
        for name in ("mi355_gemm", "mi355_layer_norm", "mi355_softmax", "mi355_index_select", "mi355_binary"):
            assert name in calls, f"{family}/{dtype}: {name} never reached ({sorted(set(calls))})"
        assert ours.dtype == plain.dtype and ours.shape == plain.shape
        tol = 2e-3 if dtype == torch.float32 else 6e-2
        err = (ours.float() - plain.float()).abs().max().item()
        scale = plain.float().abs().max().item()
        assert err <= tol * max(scale, 1.0), f"{family}/{dtype}: max abs diff {err} at scale {scale}"


def test_transposing_copy_matches_contiguous(backend):
    """`dense()` of transposed views (the copy every wrapper makes of an operand it cannot take
    as is) goes through the LDS-tiled transposing copy: bit-exact against torch's contiguous()."""
    from backendbench_amd.ops._common import copy_into, dense

    announce("transposing copy")
    g = torch.Generator().manual_seed(5)
    for dtype in (torch.float16, torch.float32, torch.int8, torch.int64, torch.bool):
        for shape in ((64, 64), (100, 37), (1000, 513), (17, 4096), (3, 130, 70), (2, 5, 65, 129),
                      (200, 136), (3, 264, 72), (1024, 520), (2, 3, 8, 4096)):   # 2-byte elements: the 16-byte form
            base = torch.randint(-100, 100, shape, generator=g).to(dtype).cuda()
            view = base.transpose(-1, -2)
            assert not view.is_contiguous()
            assert torch.equal(dense(view), view.contiguous()), (dtype, shape)
        wide = torch.randint(-100, 100, (300, 512), generator=g).to(dtype).cuda()
        view = wide[:, 7:200].t()                       # source rows longer than the part copied
        assert torch.equal(dense(view), view.contiguous()), dtype
        dst = torch.zeros(193, 400, dtype=dtype, device="cuda")[:, :300]   # destination rows longer too
        assert torch.equal(copy_into(dst, view), view)
        view = wide[:, 8:200].t()                       # the same with 16-byte aligned pieces on both sides
        dst = torch.zeros(192, 400, dtype=dtype, device="cuda")[:, 40:340]
        assert torch.equal(copy_into(dst, view), view) and torch.equal(dense(view), view.contiguous()), dtype
    # a permutation that is not a (batched) 2-D transposition keeps using the strided kernel
    x = torch.randn(6, 7, 40, 50, generator=g).cuda().permute(3, 0, 2, 1)
    assert torch.equal(dense(x), x.contiguous())
