"""The C-ABI library: it loads, exports every symbol include/mi355_aten.h declares, and the
ctypes mirror of its struct and enums matches the header.  No compute calls (no GPU here)."""

import ctypes
import os
import re

import pytest

from backendbench_amd import _lib

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "mi355_aten.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z_0-9]+)\s*\(", text)))


def header_enum(name):
    text = open(HEADER).read()
    m = re.search(r"#define\s+%s\s+(\d+)" % name, text) or re.search(r"\b%s\s*=\s*(-?\d+)" % name, text)
    assert m, name
    return int(m.group(1))


def test_header_declares_the_expected_entry_points():
    fns = declared_functions()
    assert "mi355_gemm" in fns and "mi355_softmax" in fns and "mi355_index_select" in fns
    assert len(fns) == 25


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    for fn in declared_functions():
        assert hasattr(lib, fn), f"{fn} is declared in the header but not exported"
        assert fn in _lib.SIGNATURES, f"{fn} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_abi_version_matches_header():
    assert _lib.load().mi355_abi_version() == header_enum("MI355_ABI_VERSION") == _lib.ABI_VERSION


def test_struct_layout_matches_header():
    assert header_enum("MI355_MAX_DIMS") == _lib.MAX_DIMS == 8
    assert ctypes.sizeof(_lib.TensorDesc) == 8 + 4 + 4 + 8 * 8 + 8 * 8
    assert _lib.TensorDesc.sizes.offset == 16 and _lib.TensorDesc.strides.offset == 80


@pytest.mark.parametrize("name,value", [("MI355_F32", _lib.F32), ("MI355_F16", _lib.F16), ("MI355_BF16", _lib.BF16),
                                        ("MI355_F64", _lib.F64), ("MI355_I32", _lib.I32), ("MI355_I64", _lib.I64),
                                        ("MI355_I16", _lib.I16), ("MI355_I8", _lib.I8), ("MI355_U8", _lib.U8),
                                        ("MI355_BOOL", _lib.BOOL), ("MI355_ADD", _lib.ADD), ("MI355_MUL", _lib.MUL),
                                        ("MI355_MAXIMUM", _lib.MAXIMUM), ("MI355_MINIMUM", _lib.MINIMUM), ("MI355_RELU", _lib.RELU),
                                        ("MI355_CLAMP", _lib.CLAMP), ("MI355_SUM", _lib.SUM), ("MI355_MEAN", _lib.MEAN),
                                        ("MI355_AMAX", _lib.AMAX), ("MI355_ARGMAX", _lib.ARGMAX)])
def test_enum_values_match_header(name, value):
    assert header_enum(name) == value


def test_argument_errors_are_reported_without_a_gpu():
    """Validation happens before any launch, so the error path is testable on the host."""
    lib = _lib.load()
    rc = lib.mi355_softmax(None, _lib.F32, None, _lib.F32, 4, 4, 1, 0, None, 0, None)
    assert rc == -1 and b"NULL" in lib.mi355_last_error()
    rc = lib.mi355_reduce(_lib.SUM, None, _lib.F32, 4, 0, 1, None, _lib.F32, None, 0, None)
    assert rc == -1 and b"bad extents" in lib.mi355_last_error()
    with pytest.raises(RuntimeError, match="bad extents"):
        _lib.check(rc)
    assert lib.mi355_gemm(None, 1, 1, None, 1, 1, None, 0, 0, None, 0, 8, 8, 1.0, 0.0, _lib.BF16, None, 0, None) == 0


def test_reduce_workspace_plan():
    lib = _lib.load()
    assert lib.mi355_reduce_workspace_bytes(_lib.SUM, _lib.BF16, 8192, 4096, 1) == 0      # wave per row
    assert lib.mi355_reduce_workspace_bytes(_lib.ARGMAX, _lib.F32, 8192, 128256, 1) == 0  # block per row
    ws = lib.mi355_reduce_workspace_bytes(_lib.SUM, _lib.F32, 1, 1 << 24, 1)              # one long row: split
    assert ws > 0 and ws % 4 == 0
    assert lib.mi355_reduce_workspace_bytes(_lib.ARGMAX, _lib.F32, 1, 1 << 24, 1) == ws * 4


def test_workspace_planners_run_on_the_host():
    """The two *_workspace_bytes entry points are pure host arithmetic: callable without a GPU,
    zero for shapes that are never split, and sized as splits x outputs x state otherwise."""
    lib = _lib.load()
    # reductions: many short rows need no scratch; one long row is split and needs 4-byte states
    assert lib.mi355_reduce_workspace_bytes(_lib.SUM, _lib.BF16, 8192, 4096, 1) == 0
    one_row = lib.mi355_reduce_workspace_bytes(_lib.SUM, _lib.F32, 1, 1 << 24, 1)
    assert one_row > 0 and one_row % 4 == 0 and one_row <= 4 * 4096
    arg = lib.mi355_reduce_workspace_bytes(_lib.ARGMAX, _lib.F32, 1, 1 << 24, 1)
    assert arg == 4 * one_row        # (value, int64 index) states are 16 bytes
    assert lib.mi355_reduce_workspace_bytes(_lib.SUM, _lib.F32, 0, 16, 1) == 0
    # GEMM: large outputs are never split along K; a skinny one is, in whole fp32 planes of M x N
    assert lib.mi355_gemm_workspace_bytes(4096, 4096, 11008, _lib.BF16) == 0
    skinny = lib.mi355_gemm_workspace_bytes(16, 4096, 4096, _lib.BF16)
    assert skinny > 0 and skinny % (16 * 4096 * 4) == 0 and skinny // (16 * 4096 * 4) <= 64
    assert lib.mi355_gemm_workspace_bytes(16, 4096, 4096, _lib.I32) == 0     # no integer GEMM
    assert lib.mi355_gemm_workspace_bytes(16, 4096, 32, _lib.BF16) == 0      # K too short to split
    odd = lib.mi355_gemm_workspace_bytes(24, 1001, 2048, _lib.BF16)          # rows of a plane are padded to 4 columns
    assert odd > 0 and odd % (24 * 1004 * 4) == 0
    tiny = lib.mi355_gemm_workspace_bytes(64, 250, 1040, _lib.F32)           # fp32, 64x64 tiles
    assert tiny > 0 and tiny % (64 * 252 * 4) == 0
    # 65 - 128 tiles of 256x256 with K >= 3072 (a multiple of 128): split K inside one launch, one fp32 plane
    # of 256 KB and one 8-byte flag per tile; not for fp32, a shorter K, a K off the unit, or other tile counts
    plane = 256 * 256 * 4 + 8
    assert lib.mi355_gemm_workspace_bytes(2048, 4096, 4096, _lib.BF16) == 128 * plane
    assert lib.mi355_gemm_workspace_bytes(2100, 2500, 3200, _lib.F16) == 90 * plane       # ragged tiles count whole
    assert lib.mi355_gemm_workspace_bytes(2048, 4096, 4096, _lib.F32) == 0
    assert lib.mi355_gemm_workspace_bytes(2048, 4096, 2944, _lib.BF16) == 0
    assert lib.mi355_gemm_workspace_bytes(2048, 4096, 3136, _lib.BF16) == 0
    assert lib.mi355_gemm_workspace_bytes(2304, 4096, 4096, _lib.BF16) == 0               # 144 tiles
    assert lib.mi355_gemm_workspace_bytes(4096, 4096, 4096, _lib.BF16) == 0


def _tile_columns(M, N, K=4096):
    import ctypes

    lib = _lib.load()
    wide, narrow = ctypes.c_int32(), ctypes.c_int32()
    assert lib.mi355_gemm_tile_columns(M, N, K, ctypes.byref(wide), ctypes.byref(narrow)) == 0
    return wide.value, narrow.value


def test_gemm_tile_column_plan():
    """256-wide tile columns followed by 192-wide ones when a ragged last round of tiles would idle CUs."""
    assert _tile_columns(4096, 4096) == (16, 0)            # 256 tiles: exactly one round
    assert _tile_columns(2048, 2048) == (8, 0)             # fewer tiles than CUs: nothing to balance
    assert _tile_columns(4096, 11008, 2048) == (43, 0)     # short K loop: the plain grid
    wide, narrow = _tile_columns(4096, 11008)              # 688 tiles = 2.69 rounds of 256-wide tiles
    assert narrow > 0 and 16 * wide % 256 == 0             # two full rounds, then one round of narrow tiles
    assert 16 * narrow <= 256
    for M, N in [(4096, 11008), (4104, 4500), (8192, 8192), (3000, 50257), (16384, 1000)]:
        wide, narrow = _tile_columns(M, N)
        assert wide * 256 + narrow * 192 >= N                                   # the columns cover the output
        assert narrow == 0 or wide * 256 + (narrow - 1) * 192 < N               # every narrow column starts inside it
        assert narrow > 0 or (wide - 1) * 256 < N
