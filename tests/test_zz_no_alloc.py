"""The allocation-free entry point `mi355_reduce_static` gives the results of `mi355_reduce`.

Both are called through the C ABI (ctypes) on the same inputs: `mi355_reduce` with a workspace
from torch's allocator, `mi355_reduce_static` with the buffer built into the library.  Two calls
in a row share that buffer, the second on a smaller input, so stale partial results of the
first call would show.  Bar: bit-exact (same kernels, same order of combination).
"""

import pytest
import torch

from backendbench_amd import _lib

pytestmark = pytest.mark.gpu


def _both(op, x, outer, red, inner, out_dtype):
    lib = _lib.load()
    stream = _lib.current_stream_handle()
    in_code, out_code = _lib.dtype_code(x.dtype), _lib.dtype_code(out_dtype)
    need = lib.mi355_reduce_workspace_bytes(op, in_code, outer, red, inner)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    ref = torch.empty(outer * inner, dtype=out_dtype, device=x.device)
    got = torch.full_like(ref, 77)  # poisoned: every element must be written
    _lib.check(lib.mi355_reduce(op, x.data_ptr(), in_code, outer, red, inner, ref.data_ptr(), out_code,
                                ws.data_ptr(), need, stream))
    _lib.check(lib.mi355_init())  # resolves the built-in buffer's address on this device: nothing left to ask at call time
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before, _ = torch.cuda.mem_get_info()   # hipMemGetInfo: sees every allocation on the device, not only torch's
    _lib.check(lib.mi355_reduce_static(op, x.data_ptr(), in_code, outer, red, inner, got.data_ptr(), out_code, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "mi355_reduce_static changed the device's free memory"
    return need, ref, got


@pytest.mark.parametrize("op,dtype,out_dtype", [
    (_lib.SUM, torch.float32, torch.float32),
    (_lib.AMAX, torch.bfloat16, torch.bfloat16),
    (_lib.ARGMAX, torch.float32, torch.int64),
])
def test_static_scratch_matches_workspace_form_on_two_calls_in_a_row(op, dtype, out_dtype):
    g = torch.Generator().manual_seed(5)
    big = torch.randn(3, 1 << 20, generator=g).to(dtype).cuda()      # 3 long rows: split over the chip
    small = torch.randn(2, 70001, generator=g).to(dtype).cuda()      # second call: fewer, shorter rows
    need1, ref1, got1 = _both(op, big, 3, 1 << 20, 1, out_dtype)
    need2, ref2, got2 = _both(op, small, 2, 70001, 1, out_dtype)
    assert need1 > 0 and 0 < need2 < need1, "both shapes must take the split (scratch-using) path"
    assert torch.equal(ref1, got1)
    assert torch.equal(ref2, got2)
    # and the shared kernels are right: against ATen on the CPU
    cpu = small.cpu()
    want = {_lib.SUM: lambda: cpu.sum(-1), _lib.AMAX: lambda: cpu.amax(-1), _lib.ARGMAX: lambda: cpu.argmax(-1)}[op]()
    if out_dtype == torch.int64:
        assert torch.equal(got2.cpu(), want)
    else:
        torch.testing.assert_close(got2.cpu(), want.to(out_dtype), atol=1e-2, rtol=1e-2)


def test_static_scratch_column_reduction_and_unsplit_shapes():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(2, 4096, 96, generator=g).cuda()                 # reduce the middle axis: column kernels, split
    need, ref, got = _both(_lib.SUM, x, 2, 4096, 96, torch.float32)
    assert need > 0 and torch.equal(ref, got)
    y = torch.randn(4096, 512, generator=g).cuda()                   # needs no scratch at all
    need, ref, got = _both(_lib.SUM, y, 4096, 512, 1, torch.float32)
    assert need == 0 and torch.equal(ref, got)


def test_static_scratch_refuses_what_does_not_fit():
    lib = _lib.load()
    cap = lib.mi355_reduce_static_max_bytes()
    assert cap == 4 << 20
    outer, red, inner = 1, 4096, 100000                             # 3 splits x 100000 columns x 16 B > 4 MiB
    need = lib.mi355_reduce_workspace_bytes(_lib.ARGMAX, _lib.F32, outer, red, inner)
    assert need > cap
    x = torch.zeros(8, device="cuda")
    out = torch.zeros(8, dtype=torch.int64, device="cuda")
    rc = lib.mi355_reduce_static(_lib.ARGMAX, x.data_ptr(), _lib.F32, outer, red, inner, out.data_ptr(), _lib.I64, None)
    assert rc == -1 and b"built-in buffer" in lib.mi355_last_error()


def test_static_scratch_under_graph_capture_and_replay():
    """The callers this entry point is for: recorded into a HIP graph (after mi355_init(), so the capture
    holds kernel launches only) and replayed with eager work in between; every replay gives the eager result."""
    lib = _lib.load()
    _lib.check(lib.mi355_init())
    g = torch.Generator().manual_seed(8)
    x = torch.randn(3, 1 << 20, generator=g).cuda()
    in_code = _lib.dtype_code(x.dtype)
    assert lib.mi355_reduce_workspace_bytes(_lib.SUM, in_code, 3, 1 << 20, 1) > 0
    want = torch.empty(3, device="cuda")
    _lib.check(lib.mi355_reduce_static(_lib.SUM, x.data_ptr(), in_code, 3, 1 << 20, 1, want.data_ptr(), _lib.F32,
                                       _lib.current_stream_handle()))
    torch.cuda.synchronize()
    got = torch.zeros(3, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.mi355_reduce_static(_lib.SUM, x.data_ptr(), in_code, 3, 1 << 20, 1, got.data_ptr(), _lib.F32,
                                           _lib.current_stream_handle()))
    for rep in range(4):
        got.fill_(-1.0)
        other = torch.randn(2, 70001, generator=g).cuda()          # an eager call in between shares the buffer
        tmp = torch.empty(2, device="cuda")
        _lib.check(lib.mi355_reduce_static(_lib.SUM, other.data_ptr(), in_code, 2, 70001, 1, tmp.data_ptr(), _lib.F32,
                                           _lib.current_stream_handle()))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(want, got), rep
    torch.testing.assert_close(got.cpu(), x.cpu().sum(-1), atol=1e-2, rtol=1e-2)
