"""Seeded random sweep over every functional operator slot: shapes (0-d, empty, odd sizes),
dtypes, type promotion, broadcasting and non-contiguous views drawn at random, each call
compared with the oracle (ATen on CPU copies of the same arguments).

This stands in for the reference's OpInfo suite (BackendBench/suite/opinfo.py:66-110 draws
`op_db` sample inputs per dtype), whose generator needs `expecttest`, absent from this image:
the draws below cover the same axes with a generator of our own.  Bar as in the parity tests:
integer / index / copy results bit-exact, floating point atol = rtol = 1e-2 with NaN == NaN.
"""

import os
import random
import sys

import pytest
import torch

from backendbench_amd import eval as ev
from backendbench_amd.backends import DirectoryBackend
from oracle import aten_cpu
from tight import tight_check  # noqa: E402


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
aten = torch.ops.aten
N_DRAWS = 60
SIZES = [0, 1, 1, 2, 3, 5, 8, 17, 33, 64, 130]
FLOATS = [torch.float32, torch.float16, torch.bfloat16, torch.float64]
INTS = [torch.int32, torch.int64]


@pytest.fixture(scope="module")
def backend():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return DirectoryBackend(os.path.join(ROOT, "generated_kernels"))


class Draw:
    """Random arguments from one seed; tensors are built on the CPU (identical bits both sides)."""

    def __init__(self, seed):
        self.r = random.Random(seed)
        self.g = torch.Generator().manual_seed(seed)

    def shape(self, max_rank=4, min_rank=0, zero=True):
        rank = self.r.randint(min_rank, max_rank)
        return [self.r.choice(SIZES if zero else SIZES[1:]) for _ in range(rank)]

    def dense(self, shape, dtype, scale=1.0, lo=-9, hi=10):
        if dtype.is_floating_point:
            return (torch.randn(shape, generator=self.g, dtype=torch.float32) * scale).to(dtype)
        if dtype == torch.bool:
            return torch.rand(shape, generator=self.g) > 0.5
        return torch.randint(lo, hi, shape, generator=self.g, dtype=dtype)

    def tensor(self, shape, dtype, scale=1.0, special=False):
        """A tensor of `shape`, with a randomly chosen memory layout."""
        shape = list(shape)
        kind = self.r.choice(["dense", "dense", "permuted", "strided", "offset"]) if shape else "dense"
        if kind == "permuted" and len(shape) >= 2:
            perm = list(range(len(shape)))
            self.r.shuffle(perm)
            base = self.dense([shape[p] for p in perm], dtype, scale)
            inv = [perm.index(i) for i in range(len(shape))]
            t = base.permute(inv)
        elif kind == "strided":
            big = list(shape)
            big[-1] = big[-1] * 2 + 1
            t = self.dense(big, dtype, scale)[..., 0:shape[-1] * 2:2] if shape[-1] else self.dense(shape, dtype, scale)
        elif kind == "offset":
            big = list(shape)
            big[0] = big[0] + 3
            t = self.dense(big, dtype, scale)[1:1 + shape[0]]
        else:
            t = self.dense(shape, dtype, scale)
        assert list(t.shape) == shape
        if special and dtype.is_floating_point and t.numel() and self.r.random() < 0.4:
            flat_idx = torch.randint(0, t.numel(), (max(1, t.numel() // 20),), generator=self.g)
            vals = torch.tensor([float("nan"), float("inf"), float("-inf"), 0.0, -0.0], dtype=dtype)
            pick = vals[torch.randint(0, 5, flat_idx.shape, generator=self.g)]
            idx = torch.unravel_index(flat_idx, t.shape)
            t[idx] = pick
        return t

    def broadcast_pair(self, n=2):
        full = self.shape()
        outs = []
        for _ in range(n):
            s = list(full)
            for i in range(len(s)):
                if self.r.random() < 0.25:
                    s[i] = 1
            drop = self.r.randint(0, len(s)) if self.r.random() < 0.3 else 0
            outs.append(s[drop:])
        if self.r.random() < 0.5:
            outs[0] = list(full)
        return outs

    def dtype(self, ints=True, f64=True):
        pool = FLOATS[: 4 if f64 else 3] * 2 + (INTS if ints else [])
        return self.r.choice(pool)

    def dims(self, rank):
        if rank == 0:
            return self.r.choice([[], [0], [-1]])
        k = self.r.randint(0, rank)
        ds = self.r.sample(range(rank), k)
        return [d - rank if self.r.random() < 0.5 else d for d in ds]


def _binary(op, with_alpha=False):
    def make(d):
        sa, sb = d.broadcast_pair()
        da, db = d.dtype(), d.dtype()
        kw = {}
        if with_alpha and d.r.random() < 0.5:
            both_int = not da.is_floating_point and not db.is_floating_point
            kw["alpha"] = d.r.choice([2, -3]) if both_int else d.r.choice([2, -0.5, 1.5])
        return [d.tensor(sa, da, special=True), d.tensor(sb, db, special=True)], kw
    return make


def _scalar_binary(with_alpha=False):
    def make(d):
        dt = d.dtype()
        x = d.tensor(d.shape(), dt, special=True)
        other = d.r.choice([2, -3, 0, 0.5, -1.25])
        kw = {}
        if with_alpha and d.r.random() < 0.5:
            kw["alpha"] = d.r.choice([2, -3]) if not dt.is_floating_point and isinstance(other, int) else d.r.choice([2, -0.5, 1.5])
        return [x, other], kw
    return make


def _unary(d):
    return [d.tensor(d.shape(), d.dtype(), special=True)], {}


def _clamp(d):
    dt = d.dtype()
    x = d.tensor(d.shape(), dt, special=True)
    lo, hi = sorted([d.r.uniform(-1, 1), d.r.uniform(-1, 1)]) if dt.is_floating_point else sorted([d.r.randint(-5, 5), d.r.randint(-5, 5)])
    which = d.r.choice(["both", "min", "max", "swapped"])
    if which == "min":
        return [x, lo], {}
    if which == "max":
        return [x, None, hi], {}
    if which == "swapped":
        return [x, hi, lo], {}
    return [x, lo, hi], {}


def _clamp_one(d):
    dt = d.dtype()
    b = d.r.uniform(-1, 1) if dt.is_floating_point else d.r.randint(-5, 5)
    return [d.tensor(d.shape(), dt, special=True), b], {}


def _clamp_tensor(d):
    dt = d.dtype(ints=False)
    sx, sb = d.broadcast_pair()
    full = list(torch.broadcast_shapes(sx, sb))
    x = d.tensor(full, dt, special=True)
    lo = d.tensor(sb, dt, 0.3) - 0.5 if d.r.random() < 0.8 else None
    hi = d.tensor(sb, dt, 0.3) + 0.5 if lo is None or d.r.random() < 0.6 else None
    return [x, lo, hi], {}


def _where(d):
    sc, sa, sb = d.broadcast_pair(3)
    return [d.tensor(sc, torch.bool), d.tensor(sa, d.dtype(), special=True), d.tensor(sb, d.dtype(), special=True)], {}


def _sum_dim(d):
    dt = d.dtype()
    x = d.tensor(d.shape(), dt, special=dt.is_floating_point and d.r.random() < 0.3)
    kw = {}
    if d.r.random() < 0.3:
        kw["dtype"] = d.r.choice([torch.float32, torch.float64] if dt.is_floating_point else [torch.int64, torch.float32])
    dims = d.dims(x.dim()) if d.r.random() < 0.85 else None
    return [x, dims, d.r.random() < 0.5], kw


def _mean_dim(d):
    x = d.tensor(d.shape(), d.dtype(ints=False))
    dims = d.dims(x.dim()) if d.r.random() < 0.85 else None
    return [x, dims, d.r.random() < 0.5], {}


def _full_reduce(ints):
    def make(d):
        return [d.tensor(d.shape(), d.dtype(ints=ints))], {}
    return make


def _amax(d):
    x = d.tensor(d.shape(zero=False), d.dtype(), special=True)
    return [x, d.dims(x.dim()), d.r.random() < 0.5], {}


def _argmax(d):
    dt = d.dtype()
    x = d.tensor(d.shape(zero=False), dt, special=True)
    if d.r.random() < 0.3 and x.numel():   # plant ties
        x = (x * 2).round() / 2 if dt.is_floating_point else x.clamp(-1, 1)
    if x.dim() == 0 or d.r.random() < 0.2:
        return [x], {}
    dim = d.r.randrange(-x.dim(), x.dim())
    return [x, dim, d.r.random() < 0.5], {}


def _softmax(d):
    dt = d.dtype(ints=False)
    x = d.tensor(d.shape(), dt, 2.0, special=d.r.random() < 0.3)
    dim = d.r.randrange(-x.dim(), x.dim()) if x.dim() else d.r.choice([0, -1])
    return [x, dim, dt in (torch.float16, torch.bfloat16) and d.r.random() < 0.3], {}


def _layer_norm(d):
    dt = d.dtype(ints=False)
    shape = d.shape(min_rank=1)
    if shape[-1] == 0:
        shape[-1] = 7
    k = d.r.randint(1, min(2, len(shape)))
    if any(s == 0 for s in shape[-k:]):
        k = 1
    x = d.tensor(shape, dt, 1.5) + d.r.choice([0.0, 0.0, 3.0])
    norm = shape[-k:]
    w = d.dense(norm, dt, 0.1) + 1 if d.r.random() < 0.7 else None
    b = d.dense(norm, dt, 0.1) if d.r.random() < 0.7 else None
    return [x, norm, w, b, d.r.choice([1e-5, 1e-6, 1e-3])], {}


def _mm(d):
    dt = d.r.choice([torch.bfloat16, torch.float16, torch.float32, torch.bfloat16, torch.float64])
    m, k, n = (d.r.choice([0, 1, 3, 8, 33, 64, 130, 264, 300]) for _ in range(3))
    if d.r.random() < 0.4:   # MFMA-path shapes: multiples of 8, larger
        m, k, n = d.r.choice([128, 256, 264, 520]), d.r.choice([32, 64, 96, 128, 200, 320]), d.r.choice([128, 136, 256, 512])
    a = d.dense([k, m], dt).t() if d.r.random() < 0.25 else d.dense([m, k], dt)
    b = d.dense([n, k], dt, 0.1).t() if d.r.random() < 0.4 else d.dense([k, n], dt, 0.1)
    return [a, b], {}


def _addmm(d):
    (a, b), _ = _mm(d)
    m, n = a.shape[0], b.shape[1]
    bias_shape = d.r.choice([[n], [m, n], [1, n], [m, 1], []])
    kw = {}
    if d.r.random() < 0.5:
        kw = {"beta": d.r.choice([0, 0.5, 1, -1]), "alpha": d.r.choice([1, 2.0, 0.25])}
    return [d.dense(bias_shape, a.dtype), a, b], kw


def _index_select(d):
    x = d.tensor(d.shape(min_rank=1, zero=False), d.dtype())
    dim = d.r.randrange(-x.dim(), x.dim())
    n = d.r.choice([0, 1, 4, 50])
    idx = torch.randint(0, x.shape[dim], (n,), generator=d.g, dtype=d.r.choice(INTS))
    return [x, dim, idx], {}


def _embedding(d):
    rows, width = d.r.choice([1, 7, 100]), d.r.choice([1, 8, 33, 256])
    w = d.tensor([rows, width], d.dtype(ints=False))
    idx = torch.randint(0, rows, d.shape(max_rank=3), generator=d.g, dtype=d.r.choice(INTS))
    return [w, idx] + ([d.r.choice([-1, 0])] if d.r.random() < 0.3 else []), {}


def _gather(d):
    x = d.tensor(d.shape(min_rank=1, zero=False), d.dtype())
    dim = d.r.randrange(-x.dim(), x.dim())
    ishape = [d.r.randint(0, s) if i != dim % x.dim() else d.r.choice([0, 1, 5, 40]) for i, s in enumerate(x.shape)]
    idx = torch.randint(0, x.shape[dim], ishape, generator=d.g, dtype=torch.int64)
    return [x, dim, idx], {}


SWEEP = {
    aten.add.Tensor: (_binary(aten.add.Tensor, with_alpha=True), False),
    aten.mul.Tensor: (_binary(aten.mul.Tensor), False),
    aten.add.Scalar: (_scalar_binary(with_alpha=True), False),
    aten.mul.Scalar: (_scalar_binary(), False),
    aten.clamp_min.Tensor: (_binary(aten.clamp_min.Tensor), False),   # zero ties as for maximum
    aten.clamp_max.Tensor: (_binary(aten.clamp_max.Tensor), False),
    # Not bit-exact: on a tie of -0.0 and +0.0 ATen's own CPU kernels return the second operand in
    # their vectorised loop and the first in their scalar loop; the HIP kernels follow IEEE 754-2019
    # (-0 < +0), as the GPU build of ATen does.  Values, NaN and infinities are still compared.
    aten.maximum.default: (_binary(aten.maximum.default), False),
    aten.minimum.default: (_binary(aten.minimum.default), False),
    aten.relu.default: (_unary, True),
    aten.clamp.default: (_clamp, True),
    aten.clamp_min.default: (_clamp_one, True),
    aten.clamp_max.default: (_clamp_one, True),
    aten.clamp.Tensor: (_clamp_tensor, False),
    aten.where.self: (_where, True),
    aten.sum.dim_IntList: (_sum_dim, False),
    aten.sum.default: (_full_reduce(True), False),
    aten.mean.dim: (_mean_dim, False),
    aten.mean.default: (_full_reduce(False), False),
    aten.amax.default: (_amax, False),   # the sign of a zero maximum depends on the reduction order, in ATen as here
    aten.argmax.default: (_argmax, True),
    aten._softmax.default: (_softmax, False),
    aten._log_softmax.default: (_softmax, False),
    aten.native_layer_norm.default: (_layer_norm, False),
    aten.mm.default: (_mm, False),
    aten.addmm.default: (_addmm, False),
    aten.index_select.default: (_index_select, True),
    aten.embedding.default: (_embedding, True),
    aten.gather.default: (_gather, True),
}


class _OpCase:
    def __init__(self, op):
        self.op = op


def _seed(op, i):
    return sum(map(ord, op.__name__)) * 1000 + i


def _first_differences(ref, got, limit=5):
    """Positions and values of the first elements whose bits differ, leaf by leaf."""
    out = []
    refs = ref if isinstance(ref, (tuple, list)) else [ref]
    gots = got if isinstance(got, (tuple, list)) else [got]
    for li, (a, b) in enumerate(zip(refs, gots)):
        if a.shape != b.shape or a.dtype != b.dtype:
            out.append(f"leaf {li}: {list(a.shape)} {a.dtype} vs {list(b.shape)} {b.dtype}")
            continue
        if a.numel() == 0:
            continue
        fa, fb = a.reshape(-1), b.reshape(-1)
        same = (fa == fb) | ((fa != fa) & (fb != fb))
        if a.dtype.is_floating_point:
            same &= torch.signbit(fa) == torch.signbit(fb)
        bad = (~same).nonzero().flatten()[:limit].tolist()
        out += [f"leaf {li} flat index {i}: ref {fa[i].item()!r} got {fb[i].item()!r}" for i in bad]
    return "; ".join(out)


def _describe(args, kwargs):
    def one(a):
        if isinstance(a, torch.Tensor):
            return f"T({list(a.shape)}, {str(a.dtype)[6:]}, stride={list(a.stride())})"
        return repr(a)
    return ", ".join(one(a) for a in args) + (f", {kwargs}" if kwargs else "")


@pytest.mark.parametrize("op", list(SWEEP), ids=[op.__name__ for op in SWEEP])
def test_sweep_draws_are_mostly_valid_calls(op):
    """CPU check of the generator itself: every draw builds, and ATen accepts most of them (a
    sweep of rejected calls would compare nothing)."""
    make, _ = SWEEP[op]
    accepted = 0
    for i in range(N_DRAWS):
        args, kwargs = make(Draw(_seed(op, i)))
        accepted += aten_cpu.raises(op, args, kwargs) is None
    assert accepted >= 0.8 * N_DRAWS, f"only {accepted} of {N_DRAWS} draws are valid {op.__name__} calls"


@pytest.mark.gpu
@pytest.mark.parametrize("op", list(SWEEP), ids=[op.__name__ for op in SWEEP])
def test_random_sweep_matches_the_oracle(backend, op):
    from backendbench_amd.ops import check_index_errors

    make, exact = SWEEP[op]
    impl = backend[op]
    failures = []
    for i in range(N_DRAWS):
        seed = _seed(op, i)
        args, kwargs = make(Draw(seed))
        what = f"{op.__name__} seed {seed}: {_describe(args, kwargs)}"
        print(f"\n[gpu-sweep] {what}", flush=True)
        sys.stdout.flush()
        expected_exc = None
        try:
            ref = aten_cpu.reference(op, args, kwargs)
        except Exception as exc:  # noqa: BLE001 - a draw ATen rejects must be rejected by us too
            expected_exc = type(exc)
        gpu_args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
        if expected_exc is not None:
            with pytest.raises(Exception):
                impl(*gpu_args, **kwargs)
                torch.cuda.synchronize()
                check_index_errors()
            continue
        res = impl(*gpu_args, **kwargs)
        torch.cuda.synchronize()
        check_index_errors()
        got = aten_cpu.to_cpu(res)
        if not ev.allclose(ref, got, exact=exact):
            a, r = ev.compute_errors(ref, got)
            failures.append(f"{what}\n    max abs {a}, max rel {r}\n    {_first_differences(ref, got)}")
            continue
        msg = tight_check(_OpCase(op), args, kwargs, got)   # the per-dtype bar against the fp64 restatement
        if msg is not None:
            failures.append(f"{what}\n    {msg}")
    assert not failures, f"{len(failures)} of {N_DRAWS} draws differ:\n" + "\n".join(failures)
