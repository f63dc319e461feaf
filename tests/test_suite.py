"""Suite containers and this operator set's own cases."""

import re

import torch

from backendbench_amd.suite import BaselineTestSuite, SmokeTestSuite, edge_cases, perf_cases
from backendbench_amd.suite.base import OpTest, Test as Case, TestSuite as Suite
from backendbench_amd.suite.trace import TraceTestSuite, parse_trace
from backendbench_amd.opregistry import get_operator, get_registry


def test_thunks_are_reevaluated_on_every_access():
    counter = {"n": 0}

    def thunk():
        counter["n"] += 1
        return counter["n"]

    t = Case(thunk, k=thunk)
    assert t.args == [1] and t.args == [2] and t.kwargs == {"k": 3}


def test_containers():
    ot = OpTest(torch.ops.aten.relu.default, [Case(lambda: 1)], [])
    s = Suite("mine", [ot])
    assert s.name == "mine" and list(s) == [ot] and ot.correctness_tests[0].args == [1]


def test_smoke_suite_shape():
    tests = list(SmokeTestSuite)
    assert SmokeTestSuite.name == "smoke" and len(tests) == 1 and tests[0].op is torch.ops.aten.relu.default
    (x,) = tests[0].correctness_tests[0].args
    (y,) = tests[0].performance_tests[0].args
    assert x.shape == (2,) and y.shape == (1024, 1024) and x.device.type == y.device.type == "cpu"


def test_registry_returns_canonical_objects():
    assert get_operator("add.Tensor") is torch.ops.aten.add.Tensor is get_operator(torch.ops.aten.add.Tensor)
    assert get_operator("relu") is torch.ops.aten.relu.default
    assert get_operator("definitely_not_an_op") is None
    assert "add.Tensor" in get_registry() and len(get_registry()) >= 2


def test_baseline_suite_covers_every_slot():
    from backendbench_amd.ops import SLOTS
    from backendbench_amd.utils import folder_name_to_op_name, get_pytorch_op

    suite = BaselineTestSuite("cpu", scale=0.01)
    ops = {t.op for t in suite}
    # every functional overload has suite cases; the in-place and out= overloads share their
    # kernels and are checked for aliasing and values in the GPU parity tests
    slot_ops = {get_pytorch_op(folder_name_to_op_name(f)) for f in SLOTS}
    functional = {
        op for op in slot_ops
        if not op._overloadname.endswith("out") and not op._schema.name.endswith("_")
    }
    # mm.dtype / addmm.dtype have no CPU kernel in ATen, so no suite built from the CPU oracle can hold them:
    # tests/test_variants_gpu.py checks them against the fp32 product of the widened operands
    functional -= {torch.ops.aten.mm.dtype, torch.ops.aten.addmm.dtype}
    assert len(functional) == 28 and ops == functional
    assert {c.key.split(".")[0] for c in perf_cases()} == {"C1", "C2", "C3", "C4", "C5"}
    assert len(edge_cases()) >= 250
    only = BaselineTestSuite("cpu", scale=0.01, filter=["_softmax"])
    assert [t.op for t in only] == [torch.ops.aten._softmax.default]
    t = next(iter(only)).performance_tests[0]
    a1, a2 = t.args, t.args
    assert torch.equal(a1[0], a2[0]) and a1[0] is not a2[0]   # seeded: same bits on every draw


def test_headline_work_figures():
    """Algorithmic bytes / flops per call of the measured rows."""
    w = {c.key: c.work for c in perf_cases()}
    assert w["C1.add"] == 201_326_592 and w["C1.relu"] == 134_217_728
    assert w["C2.softmax"] == 134_217_728 and w["C2.layer_norm"] == 134_299_648
    assert w["C2.sum"] == w["C2.amax"] == 67_125_248
    assert w["C3.mm_up"] == w["C3.addmm_down"] == 369_367_187_456
    assert w["C4.embedding"] == w["C4.index_select"] == 268_566_528
    assert w["C4.gather"] == 134_217_728 and w["C4.argmax"] == 4_202_758_144
    assert w["C5.mul_broadcast"] == 136_577_024 and w["C5.where_t"] == 44_040_192
    assert w["C5.maximum_t"] == 37_748_736 and w["C5.clamp_t"] == 25_165_824


def test_trace_suite(tmp_path):
    text = ("Operator: aten.relu.default\n"
            "cnt: 3, ((T([4, 8], f32),), {})\n"
            "cnt: 1, ((T([64, 8], f32),), {})\n"
            "cnt: 1, ((T([64, 8], f32),), {})\n"
            "Operator: aten.sum.SymInt\n"
            "cnt: 2, ((T([4, 8], f16), [1],), {})\n")
    entries = parse_trace(text.splitlines())
    assert [e["op_name"] for e in entries] == ["aten.relu.default"] * 3 + ["aten.sum.dim_IntList"]
    assert entries[0]["count"] == 3 and entries[0]["args"] == "((T([4, 8], f32),), {})"
    p = tmp_path / "trace.txt"
    p.write_text(text)
    suite = TraceTestSuite("t", str(p), topn=1)
    ops = list(suite)
    assert [o.op for o in ops] == [torch.ops.aten.relu.default, torch.ops.aten.sum.dim_IntList]
    tests = list(ops[0].correctness_tests)
    assert len(tests) == 1 and tests[0].args[0].shape == (64, 8)      # largest input first, duplicates merged
    assert len(list(TraceTestSuite("t", str(p), filter=["sum"]))) == 1


def test_committed_trace_fixture_parses():
    """tests/golden/transformer_block_trace.txt: 20 operators, every line a valid argument string
    whose operator resolves to one of the directory backend's slots."""
    import os

    from backendbench_amd.ops import SLOTS
    from backendbench_amd.utils import deserialize_args, op_name_to_folder_name

    path = os.path.join(os.path.dirname(__file__), "golden", "transformer_block_trace.txt")
    suite = TraceTestSuite("trace", path)
    ops = list(suite)
    assert len(ops) == 20
    n_inputs = 0
    for t in ops:
        assert op_name_to_folder_name(t.op.__name__) in SLOTS, t.op
        for text in t.inputs:
            small = re.sub(r"\d{3,}", "4", text)   # same structure, tiny extents: parse without the memory
            args, kwargs = deserialize_args(small)
            assert any(isinstance(a, torch.Tensor) for a in args)
            n_inputs += 1
    assert n_inputs == 44


def test_short_rows_trace_fixture_parses():
    """tests/golden/short_rows_and_layouts_trace.txt (the inputs of the committed kernel-trace profile of the
    short-row, transposing and fp32-tile kernels): five operators, nine inputs, one of them a strided view."""
    import os

    from backendbench_amd.ops import SLOTS
    from backendbench_amd.utils import deserialize_args, op_name_to_folder_name

    path = os.path.join(os.path.dirname(__file__), "golden", "short_rows_and_layouts_trace.txt")
    ops = list(TraceTestSuite("trace", path))
    assert len(ops) == 5 and sum(len(t.inputs) for t in ops) == 9
    strided = 0
    for t in ops:
        assert op_name_to_folder_name(t.op.__name__) in SLOTS, t.op
        for text in t.inputs:
            small = re.sub(r"\d{3,}", "4", text)
            args, _ = deserialize_args(small)
            strided += sum(isinstance(a, torch.Tensor) and not a.is_contiguous() for a in args)
    assert strided == 1
