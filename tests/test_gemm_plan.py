"""The GEMM planner's decisions, read back without a GPU.

`mi355_gemm_plan` runs `mi355_gemm`'s own dispatch (run_gemm in csrc/gemm.hip) up to the launch and
describes what it would have launched: kernel form, tile grid, parts of K and how they meet, and the
cache-warming workgroups.  These cases pin the form on both sides of the cut-offs the planner applies,
so that a change of a threshold shows up here, on the CPU, and not only as a timing on the GPU; the
results of every form are checked against the oracle by the `-m gpu` tests.
"""

import ctypes

import pytest

from backendbench_amd import _lib

CODES = {"bf16": _lib.BF16, "f16": _lib.F16, "f32": _lib.F32, "f64": _lib.F64}


def plan(M, K, N, dtype="bf16", nt=True, ws=True, a_t=False):
    """Plan of [M,K] x [K,N]; nt: b is K-contiguous (a transposed weight); a_t: a is M-contiguous."""
    lib = _lib.load()
    buf = ctypes.create_string_buffer(256)
    a_rs, a_cs = (1, M) if a_t else (K, 1)
    b_rs, b_cs = (1, K) if nt else (N, 1)
    rc = lib.mi355_gemm_plan(M, N, K, CODES[dtype], a_rs, a_cs, b_rs, b_cs, int(ws), buf, 256)
    assert rc == 0, lib.mi355_last_error()
    out = {}
    for item in buf.value.decode().split():
        k, v = item.split("=")
        out[k] = v if k in ("form", "tiles", "grid", "meet") else int(v)
    return out


def test_headline_products_run_on_the_16x16x32_kernel():
    up = plan(4096, 4096, 11008, nt=False)
    assert up["form"] == "x16_persistent" and up["tiles"] == "16x43" and up["grid"] == "256x1"
    down = plan(4096, 11008, 4096, nt=False)
    assert down["form"] == "x16" and down["grid"] == "256x1" and down["warm"] == 0
    assert plan(4096, 11008, 4096, "f16")["form"] == "x16"


@pytest.mark.parametrize("K, form", [(4096, "x16"), (4160, "w4_256x256"), (4128, "dma32_256x256"), (4104, "ktail_256x256"),
                                     (1088, "dma64_256x256"), (192, "dma64_256x256")])
def test_k_alignment_picks_the_large_tile_kernel(K, form):
    assert plan(4096, K, 4096)["form"] == form


def test_rounds_of_256x256_tiles():
    assert plan(4096, 4096, 4352)["form"] == "x16_persistent"          # 272 tiles, K >= 2048: the walk
    assert plan(4096, 1024, 4352)["form"] == "x16"                     # short K, under four rounds: one workgroup per tile
    assert plan(8192, 768, 50176)["form"] == "x16_persistent"          # 24.5 rounds
    assert plan(3072, 4096, 3072)["form"] == "x16"                     # 144 tiles: more than half the CUs
    p = plan(3072, 4096, 3072)
    assert p["warm"] == 32 and p["grid"] == "176x1"                    # ... and the idle CUs warm the cache


def test_256x128_form_between_one_round_of_128x128_and_one_of_256x128_tiles():
    p = plan(4096, 1536, 1536)
    assert p["form"] == "w4_256x128" and p["tiles"] == "16x12" and p["warm"] == 32
    assert plan(2048, 768, 2304, nt=False)["form"] == "w4_256x128"
    assert plan(2048, 768, 2048)["form"] != "w4_256x128"               # 128 tiles of 256x128: one round of 128x128 tiles
    assert plan(2048, 768, 2176)["form"] == "w4_256x128"               # 136
    p = plan(2048, 704, 2304)
    assert p["form"] == "w4_256x128" and p["warm"] == 0               # K under 768: no warming workgroups
    assert plan(2048, 256, 2304, nt=False)["form"] == "w4_256x128"
    assert plan(2048, 192, 2304)["form"] != "w4_256x128"              # K under 256
    assert plan(2048, 3072, 2304)["form"] == "w4_256x128"
    assert plan(2048, 3136, 2304)["form"] != "w4_256x128"              # K over 3072, 144 tiles
    assert plan(3840, 2048, 2048)["warm"] == 16                        # 240 tiles: 16 CUs left
    assert plan(3584, 3072, 2304, ws=False)["warm"] == 0               # 252 tiles: too few left to stay ahead
    assert plan(2048, 2048, 3712)["form"] == "w4_256x128"              # 232 tiles: close to a full round, K under 3072 ...
    assert plan(2048, 3072, 3712)["form"] == "x16_split"               # ... from there two workgroups per 256x256 tile
    assert plan(2048, 4096, 4096)["form"] == "x16_split"
    assert plan(2048, 3072, 3712, ws=False)["form"] == "w4_256x128"    # (no workspace, no split)
    p = plan(2048, 11008, 4096)
    assert p["form"] == "x16_split" and p["parts"] == 2 and p["meet"] == "inside"
    assert plan(2048, 11008, 4096, ws=False)["parts"] == 1


def test_128x128_deep_ring_and_its_split():
    p = plan(1536, 4096, 2048)
    assert p["form"] == "ring4_128x128" and p["tiles"] == "12x16" and p["parts"] == 1 and p["warm"] == 32
    assert plan(1536, 4096, 2048, nt=False)["form"] == "ring8_128x128"  # a row-major b: loader waves
    assert plan(1536, 4096, 2048, a_t=True)["form"] == "ring8_128x128"
    p = plan(1024, 11008, 1024, nt=False)
    assert p["form"] == "ring8_128x128" and p["parts"] >= 3 and p["meet"] == "inside"
    assert plan(1024, 11008, 1024, nt=False, ws=False)["parts"] == 1
    assert plan(1024, 4096, 2048)["parts"] == 2 and plan(1024, 4096, 2048)["warm"] == 0   # 128 tiles x 2 fill the chip
    p = plan(1024, 2048, 2048)                                         # ... which does not pay up to K = 2048 on a transposed b
    assert p["parts"] == 1 and p["warm"] == 32
    assert plan(1024, 2048, 2048, nt=False)["parts"] == 2
    assert plan(2048, 4128, 2048)["form"] == "small_128x128"           # K % 64 != 0: no 64-k pairs


def test_64x64_tiles_for_few_tiles_and_a_short_k():
    p = plan(768, 3072, 768, nt=False)
    assert p["form"] == "t64_ring8" and p["tiles"] == "12x12" and p["warm"] == 32
    assert plan(1024, 1024, 2048)["form"] == "t64_ring4"               # 512 tiles of 64x64: two per CU
    assert plan(1024, 2048, 2048)["form"] == "ring4_128x128"           # exactly 128 tiles of 128x128 at K = 2048
    assert plan(1024, 1536, 2048)["form"] == "t64_ring4"
    assert plan(1024, 4096, 1024)["form"] == "t64_ring8"               # 64 tiles of 128x128 up to K = 4096
    assert plan(1152, 4096, 1024)["form"].endswith("128x128")          # 72 tiles: the 128x128 kernels
    p = plan(197, 3072, 768)
    assert p["form"] == "t64_ring8" and p["parts"] > 1 and p["meet"] == "inside"
    assert plan(197, 768, 768)["parts"] == 1
    assert plan(8, 8192, 8192)["form"].endswith("128x128")             # a few rows against 134 MB of weight
    # more 64x64 tiles than CUs against a wide row-major b: the 128x128 kernels from K = 2048 on (65 - 256 rows: from 1536)
    assert plan(512, 2048, 2560)["form"] == "t64_ring4"                # (a transposed b stays)
    p = plan(512, 2048, 2560, nt=False)
    assert p["form"] == "ring8_128x128" and p["parts"] == 2 and p["meet"] == "inside"
    assert plan(512, 1536, 2560, nt=False)["form"] == "t64_ring4"
    assert plan(256, 1536, 5120, nt=False)["form"] == "ring8_128x128"
    assert plan(256, 1024, 5120, nt=False)["form"] == "t64_ring4"
    assert plan(192, 2048, 5120, nt=False)["form"] == "t64_ring8"      # 240 tiles: one per CU
    assert plan(3072, 2048, 512, nt=False)["form"] == "t64_ring4"      # a narrow b
    assert plan(64, 2048, 11008, nt=False)["form"] == "t64_ring8"      # one row of tiles


def test_other_dtypes_and_fallbacks():
    assert plan(1024, 1024, 1024, "f32")["form"] == "f32_64x64"
    assert plan(2048, 2048, 2048, "f32")["form"] == "f32_128x128_ring8"
    assert plan(4096, 4096, 4096, "f32")["form"] == "f32_128x128_ring4"
    p = plan(512, 4096, 512, "f32")
    assert p["form"] == "f32_64x64" and p["parts"] > 1 and p["meet"] == "launch"
    assert plan(1024, 4096, 1024, "f32")["parts"] == 1                  # 256 tiles of 64x64: a workgroup per CU, no split
    assert plan(512, 512, 512, "f64")["form"] == "f64_mfma"
    assert plan(2048, 100, 2048, nt=False)["form"] == "generic"         # K % 8 != 0 (the wrapper pads first)
    assert plan(2048, 1024, 1001, nt=False)["form"] == "generic"        # misaligned rows of a row-major b
    assert plan(8192, 768, 50257)["form"] == "x16"                      # a transposed b takes any N


def test_knobs_apply_to_the_plan():
    try:
        _lib.set_knob("gemm_prefetch", "0")
        assert plan(1536, 4096, 2048)["warm"] == 0
        _lib.set_knob("gemm_prefetch", "200")
        assert plan(1536, 4096, 2048)["warm"] == 64                     # cut down to the CUs left over
        _lib.set_knob("gemm_prefetch", None)
        _lib.set_knob("gemm_tile", "64x64")
        assert plan(1536, 4096, 2048)["form"].startswith("t64")
        _lib.set_knob("gemm_tile", "x16")
        assert plan(1536, 4096, 2048)["form"] == "x16"
    finally:
        _lib.set_knob("gemm_prefetch", None)
        _lib.set_knob("gemm_tile", None)
