"""The GEMM planner's own boundaries, with no knob set.

`mi355_gemm` picks one of a dozen kernel forms from the tile count, K, M and the operand layout
(run_gemm in csrc/gemm.hip).  The other GEMM tests force each form with a knob on shapes of their
choosing; this one walks shapes on both sides of every cut-off the planner itself applies -
256x256-tile counts 64/65, 96, 128/129, 191/192, 228/229, 248/249, 256/257, K = 256, 384, 1024,
2048, 3072, 4096 (a few tiles), M = 16, 64, 512, a right operand under / over 100 MB, tiles three quarters full or
less, 128/129, 224/225, 240, 256 tiles of 256x128 with K = 256 and 3072 on both sides, more 64x64 tiles than CUs
against a row-major b of 1536 columns and more with K = 1024, 1536, 2048 on both sides - and checks whatever the planner chose against the oracle.

Operands are small integers (one in four entries of a non-zero), so every sum is an integer far
inside what bf16 / f16 hold exactly and the order of summation does not matter: bit-equal to the
oracle (ATen's fp32 mm on the CPU, exact on such data) on sampled rows - the first and last row of
the matrix and both sides of every 64-, 128- and 256-row tile seam near them - over ALL columns.
"""

import os
import sys

import pytest
import torch

from backendbench_amd import eval as ev
from backendbench_amd.backends import DirectoryBackend
from oracle import aten_cpu

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
aten = torch.ops.aten


@pytest.fixture(scope="module")
def backend():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return DirectoryBackend(os.path.join(ROOT, "generated_kernels"))


def _rows(M):
    want = {0, 1, M - 1, M - 2}
    for seam in (64, 128, 256, 512):
        for base in (seam, (M // seam) * seam, (M // 2 // seam) * seam):
            want.update({base - 1, base, base + 1})
    return torch.tensor(sorted(r for r in want if 0 <= r < M))


def _check(backend, M, K, N, layout, dtype, seed, with_bias):
    g = torch.Generator(device="cuda").manual_seed(seed)     # operands drawn on the GPU: the largest is 180 M elements

    def ints(shape, lo, hi):
        return torch.randint(lo, hi, shape, generator=g, device="cuda")

    a = (ints((M, K), -1, 2) * (ints((M, K), 0, 4) == 0)).to(dtype)
    b = ints((N, K), -1, 2).to(dtype).t() if layout == "nt" else ints((K, N), -1, 2).to(dtype)
    rows = _rows(M)
    ref = aten_cpu.reference(aten.mm.default, [a[rows.cuda()].float(), b.float()])   # (the oracle copies to the CPU)
    assert float(ref.abs().max()) <= 250, "sums must stay exact in bf16"
    if with_bias:
        bias = ints((N,), -2, 3).to(dtype)
        got = backend[aten.addmm.default](bias, a, b)
        ref = ref + bias.float().cpu()
    else:
        got = backend[aten.mm.default](a, b)
    torch.cuda.synchronize()
    assert got.shape == (M, N) and got.dtype == dtype
    assert ev.bit_equal(ref.to(dtype), got[rows.cuda()].cpu()), (M, K, N, layout, dtype, "bias" if with_bias else "plain")


# (rows of 256x256 tiles, columns of tiles): the tile counts around which the planner changes kernels
_TILE_GRIDS = [(8, 8), (5, 13), (8, 12), (8, 16), (3, 43), (1, 191), (12, 16), (12, 19), (1, 229), (8, 31), (3, 83),
               (16, 16), (1, 257), (6, 16), (7, 14)]
_KS = [256, 384, 1024, 2048, 3072]


@pytest.mark.parametrize("grid", _TILE_GRIDS, ids=[f"{tm}x{tn}={tm * tn}tiles" for tm, tn in _TILE_GRIDS])
def test_planner_boundaries_in_the_tile_count(backend, grid):
    """Every K cut-off at this tile count, both layouts of b between them, whole and ragged last tiles."""
    tm, tn = grid
    print(f"\n[gpu-case] planner boundaries: {tm} x {tn} tiles of 256x256", flush=True)
    sys.stdout.flush()
    for i, K in enumerate(_KS):
        layout = "nt" if (i + tm + tn) % 2 else "nn"
        dtype = torch.bfloat16 if i % 2 == 0 else torch.float16
        ragged = i % 3 == 1                                   # last tile row / column partly filled, same tile count
        M = 256 * tm - (40 if ragged else 0)
        N = 256 * tn - (64 if ragged else 0)
        _check(backend, M, K, N, layout, dtype, seed=1000 * tm + 10 * tn + i, with_bias=(i % 2 == 1))


# Under half a round of 128x128 tiles the planner also looks at K: 64x64 tiles up to K = 4096 (at exactly 128
# tiles of 128x128 up to 2048), the 128x128 kernels with K split over the chip beyond.
_SMALL_GRIDS = [(4, 8), (2, 16), (3, 8), (2, 12), (2, 6)]


@pytest.mark.parametrize("grid", _SMALL_GRIDS, ids=[f"{tm}x{tn}={tm * tn}tiles" for tm, tn in _SMALL_GRIDS])
def test_planner_boundaries_in_k_for_a_few_tiles(backend, grid):
    tm, tn = grid
    print(f"\n[gpu-case] planner boundaries in K: {tm} x {tn} tiles of 256x256", flush=True)
    sys.stdout.flush()
    for i, K in enumerate([2048, 2112, 3072, 4096, 4160, 8192]):
        layout = "nt" if (i + tm) % 2 else "nn"
        dtype = torch.bfloat16 if (i + tn) % 2 == 0 else torch.float16
        _check(backend, 256 * tm - (24 if i % 3 == 2 else 0), K, 256 * tn, layout, dtype, seed=31 * tm + 7 * tn + i, with_bias=(i % 2 == 0))


# The 256x128 form takes 129 - 256 tiles of 256x128 (under 192 tiles of 256x256) for K = 256 .. 3072, and above
# 228 / 248 such tiles from K = 1024 on; with 16 and more CUs left over it adds cache-warming workgroups.
# (rows of 256, columns of 128): 128 / 136 / 224 / 232 / 240 / 245 / 256 tiles of 256x128
_MID_GRIDS = [(8, 16), (8, 17), (8, 28), (8, 29), (15, 16), (7, 35), (16, 16), (4, 33)]


@pytest.mark.parametrize("grid", _MID_GRIDS, ids=[f"{tm}x{tn}={tm * tn}tiles" for tm, tn in _MID_GRIDS])
def test_planner_boundaries_of_the_256x128_form(backend, grid):
    tm, tn = grid
    print(f"\n[gpu-case] planner boundaries of the 256x128 form: {tm} x {tn} tiles", flush=True)
    sys.stdout.flush()
    for i, K in enumerate([192, 256, 704, 1024, 2048, 3072, 3136]):
        layout = "nt" if (i + tm + tn) % 2 else "nn"
        dtype = torch.bfloat16 if i % 2 == 0 else torch.float16
        ragged = i % 3 == 1
        M = 256 * tm - (56 if ragged else 0)                  # (three quarters of every tile row stay output)
        N = 128 * tn - (40 if ragged else 0)
        _check(backend, M, K, N, layout, dtype, seed=900 * tm + 11 * tn + i, with_bias=(i % 2 == 0))


# More 64x64 tiles than CUs: a row-major b of 1536 and more columns moves to the 128x128 kernels from K = 2048 on
# (65 - 256 rows: from K = 1536 on), a transposed or a narrower one stays on 64x64 tiles.
@pytest.mark.parametrize("shape", [(512, 2560), (256, 5120), (320, 5120), (264, 4096), (1024, 1792), (1024, 1472), (3072, 512), (64, 11008)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_planner_boundaries_of_crowded_64x64_tiles(backend, shape):
    M, N = shape
    print(f"\n[gpu-case] planner boundaries of crowded 64x64 tiles: M = {M}, N = {N}", flush=True)
    sys.stdout.flush()
    for i, K in enumerate([1024, 1088, 1536, 1600, 2048]):
        for layout in ("nn", "nt"):
            _check(backend, M, K, N, layout, torch.bfloat16 if i % 2 == 0 else torch.float16, seed=13 * M + N + i, with_bias=(i % 2 == 1))


@pytest.mark.parametrize("M", [15, 16, 17, 63, 64, 65, 200, 180, 511, 512, 513])
def test_planner_boundaries_in_m_and_in_the_weight_size(backend, M):
    """Few rows against a wide weight: the M = 16 / 64 / 512 cut-offs, tiles more or less than three
    quarters output (M = 200 / 180 in one row of tiles), a right operand under and over 100 MB."""
    print(f"\n[gpu-case] planner boundaries: M = {M}", flush=True)
    sys.stdout.flush()
    for j, (K, N) in enumerate([(4096, 4096), (2048, 11008), (1024, 32000), (8192, 8192), (3072, 768)]):
        if K * N * 2 > 100_000_000 and M not in (16, 64, 512):
            continue                                          # the 134 MB weight at the three cut-offs only (CPU time)
        _check(backend, M, K, N, "nt" if (j + M) % 2 else "nn", torch.bfloat16, seed=77 * M + j, with_bias=(j % 2 == 0))
