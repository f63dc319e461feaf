"""Pins the oracle (oracle/aten_cpu.py = ATen on CPU) before anything is compared to it:
  1. the literal expectations of the reference's own tests
     (test/test_monkey_patch.py:100,135,188; test/test_directory_backend.py:35-94);
  2. an independent numpy float64 / integer restatement (oracle/numpy_ref.py) on every edge
     case of the suite;
  3. closed forms, invariants and brute force chosen so that a dropped term, a wrong sign or
     index, or a transposed operand fails;
  4. the committed digests in tests/golden/aten_cpu_golden.json (torch-version drift).
"""

import importlib.util
import json
import math
import os

import numpy as np
import pytest
import torch

from backendbench_amd.suite import edge_cases
from oracle import aten_cpu, numpy_ref

aten = torch.ops.aten
CASES = edge_cases()
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "aten_cpu_golden.json")


# ---- 1. literal expectations held by the reference's tests ------------------------------
def test_reference_literals():
    x = torch.tensor([-1.0, 0.0, 1.0])
    assert aten_cpu.reference(aten.relu.default, [x]).tolist() == [0.0, 0.0, 1.0]
    assert aten_cpu.reference(aten.add.Tensor, [x, torch.ones(3)]).tolist() == [0.0, 1.0, 2.0]
    assert aten_cpu.reference(aten.leaky_relu.default, [x, 0.01]).tolist() == pytest.approx([-0.01, 0.0, 1.0])
    a, b = torch.tensor([1.0, 2.0, 3.0]), torch.tensor([4.0, 5.0, 6.0])
    assert aten_cpu.reference(aten.mul.Tensor, [a, b]).tolist() == [4.0, 10.0, 18.0]
    assert aten_cpu.reference(aten.sum.default, [torch.tensor([1.0, 2.0, 3.0, 4.0])]).item() == 10.0
    assert aten_cpu.reference(aten.abs.default, [torch.tensor([-1.0, 2.0, -3.0])]).tolist() == [1.0, 2.0, 3.0]


def test_documented_special_values():
    nan, inf = float("nan"), float("inf")
    x = torch.tensor([nan, -inf, -2.0, -0.0, 0.0, 3.0, inf])
    r = aten_cpu.reference(aten.relu.default, [x])
    assert math.isnan(r[0]) and r[1:].tolist() == [0.0, 0.0, 0.0, 0.0, 3.0, inf]
    c = aten_cpu.reference(aten.clamp.default, [x, -1, 1])
    assert math.isnan(c[0]) and c[1:].tolist() == [-1.0, -1.0, 0.0, 0.0, 1.0, 1.0]
    assert aten_cpu.reference(aten.clamp.default, [torch.tensor([0.0, 5.0]), 2, 1]).tolist() == [1.0, 1.0]
    m = torch.tensor([[1, nan, 5, 5], [2, 7, 7, -inf], [inf, 1, inf, 0]])
    am = aten_cpu.reference(aten.amax.default, [m, [-1]])
    assert math.isnan(am[0]) and am[1:].tolist() == [7.0, inf]
    assert aten_cpu.reference(aten.argmax.default, [m, -1]).tolist() == [1, 1, 0]
    s = aten_cpu.reference(aten._softmax.default, [torch.tensor([[-inf, -inf], [inf, 1.0], [nan, 1.0], [-inf, 0.0]]), -1, False])
    assert torch.isnan(s[:3]).all() and s[3].tolist() == [0.0, 1.0]


# ---- 2. numpy restatement over the whole edge suite --------------------------------------
from tight import np_of, numpy_result  # noqa: E402  (shared with the GPU suites' second, tighter bar)


def tolerance(args, out):
    """Expected distance between ATen (computing in the input dtype's rules) and exact fp64."""
    dts = [x.dtype for x in args if isinstance(x, torch.Tensor) and x.dtype.is_floating_point]
    if isinstance(out, torch.Tensor) and out.dtype.is_floating_point:
        dts.append(out.dtype)
    if not dts:
        return 0.0, 0.0
    eps = max(torch.finfo(d).eps for d in dts)
    return 8 * eps, 8 * eps


@pytest.mark.parametrize("case", CASES, ids=[c.key for c in CASES])
def test_aten_cpu_matches_numpy_restatement(case):
    args, kwargs = case.make("cpu")
    if case.op.__name__ == "gather.default" and isinstance(args[0], torch.Tensor) and args[2].numel() > 20000:
        pytest.skip("brute-force gather restatement is quadratic-slow here; smaller cases cover it")
    ref = aten_cpu.reference(case.op, args, kwargs)
    want = numpy_result(case, args, kwargs)
    refs = list(ref) if isinstance(ref, (tuple, list)) else [ref]
    wants = list(want) if isinstance(want, (tuple, list)) else [want]
    assert len(refs) == len(wants)
    for r, w in zip(refs, wants):
        w = np.asarray(w)
        assert tuple(r.shape) == tuple(w.shape), (r.shape, w.shape)
        if r.dtype.is_floating_point:
            atol, rtol = tolerance(args, r)
            scale = 1.0
            n = case.op.__name__
            if n.startswith(("sum", "mean", "mm", "addmm", "native_layer_norm")):
                # accumulated rounding: bound by eps * sum |terms| rather than eps * |result|
                scale = float(np.nanmax(np.abs(w[np.isfinite(w)]))) + 64.0 if np.isfinite(w).any() else 64.0
                if n.startswith("native_layer_norm") and args[0].numel():
                    # conditioning of (x - mean) * rstd: |x| / std
                    scale += float(args[0].double().abs().max()) * float(np.max(wants[2])) * 4
            np.testing.assert_allclose(r.double().numpy(), w.astype(np.float64), rtol=rtol, atol=atol * scale, equal_nan=True)
        else:
            assert np.array_equal(r.numpy(), w.astype(r.numpy().dtype)), case.key


# ---- 3. closed forms, invariants, brute force ---------------------------------------------
def test_softmax_invariants():
    x = torch.randn(17, 333, generator=torch.Generator().manual_seed(0), dtype=torch.float64) * 3
    s = aten_cpu.reference(aten._softmax.default, [x, -1, False])
    assert torch.allclose(s.sum(-1), torch.ones(17, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(s, aten_cpu.reference(aten._softmax.default, [x + 7.25, -1, False]), atol=1e-12)  # shift
    two = aten_cpu.reference(aten._softmax.default, [torch.tensor([[0.0, math.log(3.0)]], dtype=torch.float64), -1, False])
    assert two[0].tolist() == pytest.approx([0.25, 0.75])
    assert torch.allclose(aten_cpu.reference(aten._softmax.default, [x.t().contiguous(), 0, False]), s.t())  # dim choice
    h = aten_cpu.reference(aten._softmax.default, [x.bfloat16(), -1, True])
    assert h.dtype == torch.float32 and torch.allclose(h.double(), aten_cpu.reference(aten._softmax.default, [x.bfloat16().double(), -1, False]), atol=1e-6)


def test_layer_norm_invariants():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(9, 257, generator=g, dtype=torch.float64) * 2 + 5
    w = torch.randn(257, generator=g, dtype=torch.float64) + 2
    b = torch.randn(257, generator=g, dtype=torch.float64)
    y, mean, rstd = aten_cpu.reference(aten.native_layer_norm.default, [x, [257], w, b, 1e-5])
    z = (y - b) / w
    assert torch.allclose(z.mean(-1), torch.zeros(9, dtype=torch.float64), atol=1e-10)
    assert torch.allclose(z.var(-1, unbiased=False), 1 - 1e-5 * rstd.squeeze(-1) ** 2, atol=1e-10)  # var/(var+eps)
    assert torch.allclose(mean.squeeze(-1), x.mean(-1)) and mean.shape == (9, 1)
    assert torch.allclose(rstd.squeeze(-1), 1 / torch.sqrt(x.var(-1, unbiased=False) + 1e-5))
    const = torch.full((2, 8), 3.0, dtype=torch.float64)
    y, mean, rstd = aten_cpu.reference(aten.native_layer_norm.default, [const, [8], None, None, 0.25])
    assert y.abs().max() == 0 and mean.flatten().tolist() == [3.0, 3.0] and rstd.flatten().tolist() == [2.0, 2.0]
    # f16/bf16 inputs: statistics come back in fp32 and equal the statistics of the upcast input
    xb = x.bfloat16()
    _, m32, r32 = aten_cpu.reference(aten.native_layer_norm.default, [xb, [257], None, None, 1e-5])
    assert m32.dtype == r32.dtype == torch.float32
    assert torch.allclose(m32.squeeze(-1).double(), xb.double().mean(-1), atol=1e-5)


def test_matmul_identities():
    g = torch.Generator().manual_seed(2)
    a = torch.randn(7, 5, generator=g, dtype=torch.float64)
    b = torch.randn(5, 3, generator=g, dtype=torch.float64)
    c = torch.randn(3, generator=g, dtype=torch.float64)
    mm = aten_cpu.reference(aten.mm.default, [a, b])
    brute = torch.tensor([[sum(a[i, k].item() * b[k, j].item() for k in range(5)) for j in range(3)] for i in range(7)], dtype=torch.float64)
    assert torch.allclose(mm, brute, atol=1e-12)
    assert not torch.allclose(mm, aten_cpu.reference(aten.mm.default, [a, b.flip(0)]))          # k order matters
    assert torch.equal(aten_cpu.reference(aten.mm.default, [torch.eye(5, dtype=torch.float64), b]), b)
    onehot = torch.zeros(2, 5, dtype=torch.float64)
    onehot[0, 3] = onehot[1, 0] = 1
    assert torch.equal(aten_cpu.reference(aten.mm.default, [onehot, b]), b[[3, 0]])                # row selection
    assert torch.allclose(aten_cpu.reference(aten.addmm.default, [c, a, b], {"beta": 0.5, "alpha": 2.0}), 0.5 * c + 2 * mm)
    nanc = torch.full((3,), float("nan"), dtype=torch.float64)
    assert torch.allclose(aten_cpu.reference(aten.addmm.default, [nanc, a, b], {"beta": 0, "alpha": 3.0}), 3 * mm)
    assert aten_cpu.reference(aten.mm.default, [torch.zeros(2, 0), torch.zeros(0, 3)]).tolist() == [[0.0] * 3] * 2


def test_reduction_closed_forms():
    v = [0.1 * i - 3 for i in range(101)]
    x = torch.tensor(v, dtype=torch.float64)
    assert aten_cpu.reference(aten.sum.default, [x]).item() == pytest.approx(math.fsum(v), abs=1e-12)
    assert aten_cpu.reference(aten.mean.default, [x]).item() == pytest.approx(math.fsum(v) / 101, abs=1e-12)
    ar = torch.arange(1, 101, dtype=torch.int32).reshape(4, 25)
    s = aten_cpu.reference(aten.sum.dim_IntList, [ar, [-1]])
    assert s.dtype == torch.int64 and s.tolist() == [sum(range(1 + 25 * r, 26 + 25 * r)) for r in range(4)]
    g = torch.Generator().manual_seed(3)
    y = torch.randn(13, 77, generator=g)
    idx = aten_cpu.reference(aten.argmax.default, [y, -1])
    assert torch.equal(aten_cpu.reference(aten.amax.default, [y, [-1]]), y.gather(1, idx[:, None]).squeeze(1))
    ties = torch.tensor([[1.0, 3.0, 3.0, 2.0], [5.0, 5.0, 5.0, 5.0]])
    assert aten_cpu.reference(aten.argmax.default, [ties, -1]).tolist() == [1, 0]                    # first index wins
    assert aten_cpu.reference(aten.argmax.default, [ties]).item() == 4                              # flattened
    assert aten_cpu.raises(aten.mean.dim, [ar, [-1]]) is RuntimeError
    assert aten_cpu.raises(aten.amax.default, [torch.zeros(4, 0), [-1]]) is IndexError
    assert math.isnan(aten_cpu.reference(aten.mean.dim, [torch.zeros(4, 0), [-1]])[0].item())


def test_indexing_brute_force():
    g = torch.Generator().manual_seed(4)
    table = torch.randn(11, 6, generator=g)
    idx = torch.randint(0, 11, (2, 5), generator=g)
    emb = aten_cpu.reference(aten.embedding.default, [table, idx])
    assert emb.shape == (2, 5, 6)
    for i in range(2):
        for j in range(5):
            assert torch.equal(emb[i, j], table[idx[i, j]])
    assert torch.equal(emb.reshape(10, 6), aten_cpu.reference(aten.index_select.default, [table, 0, idx.reshape(-1)]))
    cols = torch.randint(0, 6, (4,), generator=g)
    sel = aten_cpu.reference(aten.index_select.default, [table, 1, cols])
    assert all(torch.equal(sel[:, j], table[:, cols[j]]) for j in range(4))
    gi = torch.randint(0, 6, (11, 3), generator=g)
    ga = aten_cpu.reference(aten.gather.default, [table, 1, gi])
    assert all(ga[i, j] == table[i, gi[i, j]] for i in range(11) for j in range(3))
    g0 = torch.randint(0, 11, (4, 6), generator=g)
    gb = aten_cpu.reference(aten.gather.default, [table, 0, g0])
    assert all(gb[i, j] == table[g0[i, j], j] for i in range(4) for j in range(6))
    assert aten_cpu.raises(aten.index_select.default, [table, 0, torch.tensor([11])]) is IndexError
    assert aten_cpu.raises(aten.index_select.default, [table, 0, torch.tensor([-1])]) is IndexError
    assert aten_cpu.raises(aten.gather.default, [table, 1, torch.tensor([[-1]])]) is RuntimeError


def test_elementwise_scalar_definitions():
    g = torch.Generator().manual_seed(5)
    a, b = torch.randn(50, generator=g, dtype=torch.float64), torch.randn(50, generator=g, dtype=torch.float64)
    cond = a > 0
    assert aten_cpu.reference(aten.add.Tensor, [a, b], {"alpha": -2.5}).tolist() == pytest.approx(
        [x - 2.5 * y for x, y in zip(a.tolist(), b.tolist())], rel=1e-15)  # fused vs separate rounding
    assert aten_cpu.reference(aten.add.Tensor, [a, b]).tolist() == [x + y for x, y in zip(a.tolist(), b.tolist())]
    assert aten_cpu.reference(aten.mul.Tensor, [a, b]).tolist() == [x * y for x, y in zip(a.tolist(), b.tolist())]
    assert aten_cpu.reference(aten.maximum.default, [a, b]).tolist() == [max(x, y) for x, y in zip(a.tolist(), b.tolist())]
    assert aten_cpu.reference(aten.where.self, [cond, a, b]).tolist() == [x if c else y for c, x, y in zip(cond.tolist(), a.tolist(), b.tolist())]
    assert aten_cpu.reference(aten.clamp.default, [a, -0.5, 0.25]).tolist() == [min(max(x, -0.5), 0.25) for x in a.tolist()]
    # promotion rules the wrappers have to reproduce
    f16, f32, f64 = torch.float16, torch.float32, torch.float64
    assert aten_cpu.reference(aten.add.Tensor, [torch.ones(2, dtype=f16), torch.ones(2, dtype=f32)]).dtype == f32
    assert aten_cpu.reference(aten.add.Tensor, [torch.ones(2, dtype=f16), torch.tensor(1.0, dtype=f64)]).dtype == f16
    assert aten_cpu.reference(aten.add.Tensor, [torch.ones(2, dtype=torch.int32), torch.tensor(1.0)]).dtype == f32
    assert aten_cpu.reference(aten.where.self, [torch.tensor([True]), torch.ones(1, dtype=f16), torch.ones(1)]).dtype == f32


# ---- 4. golden digests (drift of the torch build) --------------------------------------------
def _digest_module():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(GOLDEN), "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_golden_file_covers_every_case():
    table = json.load(open(GOLDEN))
    assert sorted(table["cases"]) == sorted(c.key for c in CASES)


@pytest.mark.parametrize("case", CASES, ids=[c.key for c in CASES])
def test_oracle_matches_golden(case):
    table = json.load(open(GOLDEN))["cases"]
    got = _digest_module().record(case)
    want = table[case.key]
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert g["shape"] == w["shape"] and g["dtype"] == w["dtype"]
        if "sha256" in w:
            assert g["sha256"] == w["sha256"]
        else:
            assert (g["nan"], g["pinf"], g["ninf"]) == (w["nan"], w["pinf"], w["ninf"])
            assert g["l1"] == pytest.approx(w["l1"], rel=2e-3, abs=1e-3)
            assert g["total"] == pytest.approx(w["total"], rel=2e-3, abs=2e-3 * max(1.0, w["l1"]))


# ---- 5. the tighter per-dtype bar tells accumulator widths apart (CPU mock of the comparer) -----------
class _Case:
    def __init__(self, op):
        self.op = op


def _narrow_sum(terms, dtype, chunk=128):
    """Sum along the last axis in chunks of `chunk` terms (each chunk in fp32) with the running total rounded
    to `dtype` after every chunk: an accumulator that is only partly as wide as advertised."""
    acc = torch.zeros(terms.shape[:-1], dtype=dtype)
    for i in range(0, terms.shape[-1], chunk):
        acc = (acc.float() + terms[..., i : i + chunk].float().sum(-1)).to(dtype)
    return acc


def test_tight_bar_separates_fp32_from_bf16_accumulation():
    from tight import tight_check

    g = torch.Generator().manual_seed(3)
    a = torch.randn(8, 512, generator=g).bfloat16()
    b = (torch.randn(512, 6, generator=g) * 0.02).bfloat16()
    case = _Case(aten.mm.default)
    terms = a.float()[:, None, :] * b.float().t()[None, :, :]          # [8, 6, 512] exact products
    fp32_acc = terms.sum(-1).bfloat16()
    bf16_acc = _narrow_sum(terms, torch.bfloat16)
    assert ev_allclose(fp32_acc, bf16_acc)                              # the reference's 1e-2 bar sees no difference
    assert tight_check(case, [a, b], {}, fp32_acc) is None
    assert "mm.default" in tight_check(case, [a, b], {}, bf16_acc)
    # fp32 results: an fp32 accumulator passes, an f16 one does not
    af, bf_ = torch.randn(4, 2048, generator=g), torch.randn(2048, 3, generator=g)
    t32 = af[:, None, :] * bf_.t()[None, :, :]
    assert tight_check(case, [af, bf_], {}, t32.sum(-1)) is None
    assert tight_check(case, [af, bf_], {}, _narrow_sum(t32, torch.float16).float()) is not None


def test_tight_bar_separates_fp64_from_fp32_arithmetic():
    from tight import tight_check

    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 300, generator=g, dtype=torch.float64) * 3
    sm = _Case(aten._softmax.default)
    assert tight_check(sm, [x, -1, False], {}, torch.softmax(x, -1)) is None
    assert tight_check(sm, [x, -1, False], {}, torch.softmax(x.float(), -1).double()) is not None
    ln = _Case(aten.native_layer_norm.default)
    w, b = torch.randn(300, generator=g, dtype=torch.float64), torch.randn(300, generator=g, dtype=torch.float64)
    good = torch.ops.aten.native_layer_norm(x, [300], w, b, 1e-5)
    assert tight_check(ln, [x, [300], w, b, 1e-5], {}, good) is None
    low = tuple(t.double() for t in torch.ops.aten.native_layer_norm(x.float(), [300], w.float(), b.float(), 1e-5))
    assert tight_check(ln, [x, [300], w, b, 1e-5], {}, low) is not None
    # half outputs: one rounding of the fp32 result passes, a second rounding through a coarser type does not
    xs = torch.randn(64, 1000, generator=g).bfloat16()
    sm_out = torch.softmax(xs.float(), -1)
    assert tight_check(sm, [xs, -1, False], {}, sm_out.bfloat16()) is None
    assert tight_check(sm, [xs, -1, False], {}, (sm_out * 1.02).bfloat16()) is not None   # 2 % off: inside 1e-2 + 1e-2 |x|
    sums = _Case(aten.sum.dim_IntList)
    big = (torch.randn(16, 4096, generator=g) * 4).bfloat16()
    assert tight_check(sums, [big, [-1]], {}, big.float().sum(-1).bfloat16()) is None
    assert tight_check(sums, [big, [-1]], {}, _narrow_sum(big, torch.bfloat16)) is not None


def ev_allclose(a, b):
    from backendbench_amd import eval as ev

    return ev.allclose(a, b)
