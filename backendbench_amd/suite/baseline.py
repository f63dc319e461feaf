"""The operator set's own test suite: headline shapes plus edge layouts.

The reference's OpInfo / TorchBench / FACTO suites (BackendBench/suite/opinfo.py,
torchbench.py, facto.py) need packages or downloads this environment does not have, so
this module is the input source for the operator slots: `perf_cases()` are the
headline configurations (one per measured row: shapes, dtypes, distributions and the
algorithmic bytes / flops used for roofline fractions) and `edge_cases()` are small
inputs covering broadcasting, non-contiguous views, NaN / +-inf, ties, empty and 0-d
tensors, integer dtypes and argument variants.  Every tensor is drawn on the CPU from a
seeded generator and then moved, so any two devices see identical bits.
"""

from dataclasses import dataclass, field
from typing import Callable, Dict, List

import torch

from ..opregistry import get_operator
from .base import OpTest, Test, TestSuite

aten = torch.ops.aten


@dataclass
class Case:
    key: str                 # e.g. "C2.softmax"
    op: object               # OpOverload
    make: Callable           # device -> (args, kwargs)
    work: float = 0.0        # algorithmic bytes (bound == "hbm") or flops ("mfma") per call
    bound: str = "hbm"
    exact: bool = False      # outputs must be bit-identical to the reference
    note: str = ""
    extra: Dict = field(default_factory=dict)


def _gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def normal(shape, dtype, mean=0.0, std=1.0, seed=0):
    """N(mean, std) drawn in fp32 on the CPU, rounded once to `dtype`."""
    t = torch.empty(shape, dtype=torch.float32)
    t.normal_(mean, std, generator=_gen(seed))
    return t.to(dtype)


def randint(shape, high, seed=0, dtype=torch.int64, low=0):
    return torch.randint(low, high, shape, generator=_gen(seed), dtype=dtype)


def poison(t, frac=0.01, seed=0):
    """Set `frac` of the elements to NaN, +inf, -inf (a third each) at seeded positions."""
    flat = t.reshape(-1)
    n = flat.numel()
    k = max(3, int(n * frac)) if n >= 3 else 0
    if k == 0:
        return t
    pos = torch.randperm(n, generator=_gen(seed))[:k]
    third = k // 3
    flat[pos[:third]] = float("nan")
    flat[pos[third : 2 * third]] = float("inf")
    flat[pos[2 * third :]] = float("-inf")
    return t


def _to(device, *tensors):
    return [t.to(device) if isinstance(t, torch.Tensor) else t for t in tensors]


# ---------------------------------------------------------------- headline configurations
def perf_cases(scale: float = 1.0) -> List[Case]:
    """One Case per measured row.  `scale` < 1 shrinks the leading extent of every shape
    (same kernels, same layouts) for quick runs on small machines."""

    def S(n, mult=1):
        return max(mult, int(n * scale) // mult * mult)

    bf16, f16, f32 = torch.bfloat16, torch.float16, torch.float32
    cases = []

    # C1: add.Tensor then relu, fp32 contiguous [4096, 4096]
    m1 = S(4096)
    cases.append(Case("C1.add", aten.add.Tensor,
                      lambda d: (_to(d, normal((m1, 4096), f32, seed=1), normal((m1, 4096), f32, seed=2)), {}),
                      work=3 * 4 * m1 * 4096))
    cases.append(Case("C1.relu", aten.relu.default,
                      lambda d: (_to(d, normal((m1, 4096), f32, seed=1) + normal((m1, 4096), f32, seed=2)), {}),
                      work=2 * 4 * m1 * 4096, note="input is the C1 add result"))

    # C2: row ops on bf16 [8192, 4096], N(0, 2)
    m2, n2 = S(8192), 4096
    x2 = lambda: normal((m2, n2), bf16, 0.0, 2.0, seed=3)
    cases.append(Case("C2.softmax", aten._softmax.default, lambda d: (_to(d, x2(), -1, False), {}),
                      work=2 * 2 * m2 * n2))
    cases.append(Case("C2.layer_norm", aten.native_layer_norm.default,
                      lambda d: (_to(d, x2(), [n2], normal((n2,), bf16, 1.0, 0.1, seed=4),
                                     normal((n2,), bf16, 0.0, 0.1, seed=5), 1e-5), {}),
                      work=2 * 2 * m2 * n2 + 2 * 2 * n2 + 2 * 4 * m2))
    cases.append(Case("C2.sum", aten.sum.dim_IntList, lambda d: (_to(d, x2(), [-1]), {}),
                      work=2 * m2 * n2 + 2 * m2))
    cases.append(Case("C2.amax", aten.amax.default, lambda d: (_to(d, x2(), [-1]), {}),
                      work=2 * m2 * n2 + 2 * m2))

    # C3: mm / addmm, bf16, 7B MLP shapes
    m3 = S(4096, 256)
    for tag, (K, N) in (("up", (4096, 11008)), ("down", (11008, 4096))):
        a = lambda K=K: normal((m3, K), bf16, seed=6)
        b = lambda K=K, N=N: normal((K, N), bf16, 0.0, 0.02, seed=7)
        flops = 2.0 * m3 * N * K
        cases.append(Case(f"C3.mm_{tag}", aten.mm.default, lambda d, a=a, b=b: (_to(d, a(), b()), {}),
                          work=flops, bound="mfma", extra={"bytes": 2 * (m3 * K + K * N + m3 * N)}))
        cases.append(Case(f"C3.addmm_{tag}", aten.addmm.default,
                          lambda d, a=a, b=b, N=N: (_to(d, normal((N,), bf16, 0.0, 0.02, seed=8), a(), b()), {}),
                          work=flops, bound="mfma", extra={"bytes": 2 * (m3 * K + K * N + m3 * N + N)}))

    # C4: indexing, bit-exact
    v4, d4, n4 = S(128256), 4096, S(16384)
    table = lambda: normal((v4, d4), bf16, 0.0, 0.02, seed=9)
    idx = lambda: randint((n4,), v4, seed=10)
    cases.append(Case("C4.embedding", aten.embedding.default, lambda d: (_to(d, table(), idx()), {}),
                      work=2 * 2 * n4 * d4 + 8 * n4, exact=True))
    cases.append(Case("C4.index_select", aten.index_select.default, lambda d: (_to(d, table(), 0, idx()), {}),
                      work=2 * 2 * n4 * d4 + 8 * n4, exact=True))
    g4 = S(2048)
    cases.append(Case("C4.gather", aten.gather.default,
                      lambda d: (_to(d, normal((g4, 4096), f32, seed=11), 1, randint((g4, 4096), 4096, seed=12)), {}),
                      work=(4 + 8 + 4) * g4 * 4096, exact=True))
    r4 = S(8192)
    cases.append(Case("C4.argmax", aten.argmax.default,
                      lambda d: (_to(d, normal((r4, 128256), f32, seed=13), -1), {}),
                      work=4 * r4 * 128256 + 8 * r4, exact=True))

    # C5: fp16 edge layouts with 1 % NaN / +-inf
    b5 = S(64)
    cases.append(Case("C5.mul_broadcast", aten.mul.Tensor,
                      lambda d: (_to(d, normal((b5, 1, 2048), f16, seed=14), normal((1, 512, 2048), f16, seed=15)), {}),
                      work=2 * (b5 * 512 * 2048 + b5 * 2048 + 512 * 2048)))
    r5 = S(2048)
    base = lambda seed: poison(normal((r5, 3072), f16, seed=seed), 0.01, seed=seed + 100)

    def tview(device, seed):
        return base(seed).to(device).t()  # [3072, r5] view with strides (1, 3072)

    def cond_t(device):
        return (normal((r5, 3072), f32, seed=19) > 0).to(device).t()

    cases.append(Case("C5.where_t", aten.where.self, lambda d: ([cond_t(d), tview(d, 16), tview(d, 17)], {}),
                      work=(1 + 2 + 2 + 2) * r5 * 3072, exact=True))
    cases.append(Case("C5.maximum_t", aten.maximum.default, lambda d: ([tview(d, 16), tview(d, 17)], {}),
                      work=3 * 2 * r5 * 3072))
    cases.append(Case("C5.clamp_t", aten.clamp.default, lambda d: ([tview(d, 16), -1, 1], {}),
                      work=2 * 2 * r5 * 3072))
    return cases


# ---------------------------------------------------------------- edge cases
def edge_cases() -> List[Case]:
    bf16, f16, f32, f64 = torch.bfloat16, torch.float16, torch.float32, torch.float64
    i32, i64 = torch.int32, torch.int64
    C: List[Case] = []
    n = [0]

    def add(op, make, exact=False, tag="", stock_gpu=True):
        # stock_gpu=False: ATen's own GPU kernel refuses these arguments (bf16 half_to_float, fp32
        # gamma / beta on a half input) although its CPU kernel and ours take them; suites built for
        # a GPU leave the case out, because the evaluator computes its reference with the stock op
        n[0] += 1
        name = op.__name__.replace(".", "_")
        C.append(Case(f"E{n[0]:03d}.{name}{('.' + tag) if tag else ''}", op, make, exact=exact,
                      extra={} if stock_gpu else {"cpu_reference_only": True}))

    special = lambda dt: torch.tensor([float("nan"), float("-inf"), -2.0, -0.0, 0.0, 3.0, float("inf"), 0.5], dtype=dt)

    # ---- binary: add / mul / maximum
    for op in (aten.add.Tensor, aten.mul.Tensor, aten.maximum.default, aten.minimum.default):
        for dt in (f32, f16, bf16):
            add(op, lambda d, dt=dt: (_to(d, normal((33, 65), dt, seed=1), normal((33, 65), dt, seed=2)), {}), tag=f"{dt}".split(".")[-1])
        add(op, lambda d: (_to(d, normal((4, 1, 16), f16, seed=3), normal((1, 5, 16), f16, seed=4)), {}), tag="bcast3")
        add(op, lambda d: (_to(d, normal((7, 1), f32, seed=3), normal((1, 9), f32, seed=4)), {}), tag="outer")
        add(op, lambda d: (_to(d, normal((6, 40), f32, seed=3), normal((40,), f32, seed=4)), {}), tag="rowvec")
        add(op, lambda d: ([normal((48, 20), f16, seed=5).to(d).t(), normal((48, 20), f16, seed=6).to(d).t()], {}), tag="both_t")
        add(op, lambda d: ([normal((48, 20), f32, seed=5).to(d).t(), normal((20, 48), f32, seed=6).to(d)], {}), tag="mixed_layout")
        add(op, lambda d: ([normal((16, 64), f32, seed=5).to(d)[:, ::2], normal((16, 32), f32, seed=6).to(d)], {}), tag="strided")
        add(op, lambda d: (_to(d, poison(normal((50, 30), f16, seed=7), 0.05, 8), poison(normal((50, 30), f16, seed=9), 0.05, 10)), {}), tag="naninf")
        add(op, lambda d: (_to(d, special(f32), special(f32).flip(0)), {}), tag="special")
        add(op, lambda d: (_to(d, torch.empty(0, 128, dtype=f16), torch.empty(0, 128, dtype=f16)), {}), tag="empty")
        add(op, lambda d: (_to(d, torch.empty(0, 128, dtype=f16), normal((128,), f16, seed=1)), {}), tag="empty_bcast")
        add(op, lambda d: (_to(d, torch.tensor(1.5, dtype=f16), torch.tensor(-2.25, dtype=f16)), {}), tag="0d")
        add(op, lambda d: (_to(d, normal((5, 3), f32, seed=1), torch.tensor(2.0, dtype=f32)), {}), tag="0d_bcast")
        add(op, lambda d: (_to(d, normal((9,), f16, seed=1), normal((9,), f32, seed=2)), {}), tag="promote_f16_f32")
        add(op, lambda d: (_to(d, normal((9,), f16, seed=1), torch.tensor(0.5, dtype=f64)), {}), tag="promote_0d_f64")
        add(op, lambda d: (_to(d, randint((9,), 100, 1, i32, -100), torch.tensor(0.5, dtype=f32)), {}), tag="promote_int_0d_f32")
        add(op, lambda d: (_to(d, randint((17, 5), 100, 1, i64, -100), randint((17, 5), 100, 2, i64, -100)), {}), exact=True, tag="i64")
        add(op, lambda d: (_to(d, randint((17, 5), 100, 1, i32, -100), randint((5,), 100, 2, i32, -100)), {}), exact=True, tag="i32")
        add(op, lambda d: (_to(d, normal((4, 6), f64, seed=1), normal((4, 6), f64, seed=2)), {}), tag="f64")
        add(op, lambda d: (_to(d, normal((3, 1000, 7), bf16, seed=1), normal((3, 1000, 7), bf16, seed=2)), {}), tag="odd_inner")
    add(aten.add.Tensor, lambda d: (_to(d, normal((33, 65), f32, seed=1), normal((33, 65), f32, seed=2)), {"alpha": 2.5}), tag="alpha")
    add(aten.add.Tensor, lambda d: (_to(d, normal((33, 65), bf16, seed=1), normal((65,), bf16, seed=2)), {"alpha": -1}), tag="alpha_bf16")
    add(aten.add.Tensor, lambda d: (_to(d, randint((12,), 50, 1, i64), randint((12,), 50, 2, i64)), {"alpha": 3}), exact=True, tag="alpha_int")
    # dense output, innermost extent no multiple of the vector width, one operand broadcast or strided: vector
    # stores over the flat output, the odd operand gathered along a coordinate walk (attention map + mask at 197 tokens)
    add(aten.add.Tensor, lambda d: (_to(d, normal((2, 3, 197, 197), f16, seed=1), normal((2, 1, 1, 197), f16, seed=2)), {}), tag="mask_197_f16")
    add(aten.mul.Tensor, lambda d: (_to(d, poison(normal((33, 131), f32, seed=1), 0.01, 3), normal((131,), f32, seed=2)), {}), tag="row_131_f32")
    add(aten.add.Tensor, lambda d: (_to(d, normal((3, 1367), bf16, seed=1), normal((1367,), bf16, seed=2)), {"alpha": 0.5}), tag="ragged_tail_bf16")
    add(aten.where.self, lambda d: (_to(d, normal((5, 1, 77), f32, seed=1) > 0, normal((5, 19, 77), f16, seed=2), normal((1, 19, 1), f16, seed=3)), {}), exact=True, tag="three_way_77")
    add(aten.maximum.default, lambda d: ([normal((67, 65), f32, seed=1).to(d), normal((65, 67), f32, seed=2).to(d).t()], {}), tag="transposed_odd")
    # Scalar overloads and the tensor-bound one-sided clamps
    add(aten.add.Scalar, lambda d: ([normal((33, 65), bf16, seed=1).to(d), 1.5], {"alpha": 2}), tag="bf16_alpha")
    add(aten.add.Scalar, lambda d: ([randint((6, 10), 50, 1, i32).to(d), 2.5], {}), tag="int_plus_float")
    add(aten.mul.Scalar, lambda d: ([normal((128, 130), f16, seed=1).to(d), 0.125], {}), tag="f16")
    add(aten.mul.Scalar, lambda d: ([randint((6, 10), 50, 1, i64).to(d), 3], {}), exact=True, tag="int")
    add(aten.clamp_min.Tensor, lambda d: ([poison(normal((40, 24), f32, seed=1), 0.05, 3).to(d), normal((24,), f32, seed=2).to(d)], {}), tag="bcast_naninf")
    add(aten.clamp_max.Tensor, lambda d: ([normal((40, 24), bf16, seed=1).to(d), normal((40, 1), bf16, seed=2).to(d)], {}), tag="bcast_col_bf16")
    # one operand the transpose of the other's layout: large matrices are re-laid first, small or batched ones read in place
    add(aten.add.Tensor, lambda d: ([normal((1100, 1030), f32, seed=1).to(d), normal((1030, 1100), f32, seed=2).to(d).t()], {}), tag="mixed_layout_large")
    add(aten.add.Tensor, lambda d: ([normal((8, 48, 48, 96), f16, seed=1).to(d).permute(0, 3, 1, 2), normal((8, 96, 48, 48), f16, seed=2).to(d)], {}), tag="channels_last_view_plus_dense_large")
    add(aten.maximum.default, lambda d: ([normal((6, 300, 520), f32, seed=1).to(d), normal((520, 6, 300), f32, seed=2).to(d).permute(1, 2, 0)], {}), tag="rotated_dims_large")
    add(aten.mul.Tensor, lambda d: ([normal((4, 6, 64, 197), f16, seed=1).to(d).transpose(-1, -2), normal((4, 6, 197, 64), f16, seed=2).to(d)], {}), tag="mixed_layout_heads")
    add(aten.where.self, lambda d: ([cond((900, 1200), 1).to(d), normal((1200, 900), f16, seed=2).to(d).t(), normal((900, 1200), f16, seed=3).to(d)], {}), exact=True, tag="mixed_layout_large")
    add(aten.add.Tensor, lambda d: (_to(d, normal((7, 599), f16, seed=1), normal((7, 599), f32, seed=2)), {}), tag="promote_odd")
    add(aten.mul.Tensor, lambda d: ([normal((9, 1001), f32, seed=1).to(d)[:, ::2], normal((501,), f32, seed=2).to(d)], {}), tag="strided_cols_odd")
    add(aten.clamp.Tensor, lambda d: (_to(d, normal((11, 401), f32, seed=1), normal((401,), f32, -0.5, 0.1, seed=2), normal((11, 1), f32, 0.5, 0.1, seed=3)), {}), tag="bounds_broadcast_odd")
    # fp32 with f16 / bf16: the narrow operand is widened inside the kernel
    add(aten.mul.Tensor, lambda d: (_to(d, normal((33, 64), f32, seed=1), normal((64,), bf16, seed=2)), {}), tag="f32_times_bf16_row")
    add(aten.add.Tensor, lambda d: ([normal((40, 24), f16, seed=1).to(d).t(), normal((24, 40), f32, seed=2).to(d)], {"alpha": -1.5}), tag="f16_t_plus_f32_alpha")
    add(aten.mul.Tensor, lambda d: (_to(d, poison(normal((5, 0, 3), bf16, seed=1), 0.0, 1), normal((5, 1, 3), f32, seed=2)), {}), tag="mixed_empty")
    add(aten.add.Tensor, lambda d: (_to(d, poison(normal((4100,), f16, seed=1), 0.01, 3), normal((4100,), f32, seed=2)), {}), tag="mixed_flat_specials")
    # channels-last operand with a per-channel broadcast: the kernel walks the dims in the output's memory order
    add(aten.mul.Tensor, lambda d: ([normal((6, 40, 9, 7), f16, seed=1).to(d).to(memory_format=torch.channels_last), normal((1, 40, 1, 1), f16, seed=2).to(d)], {}), tag="channels_last_scale")
    add(aten.add.Tensor, lambda d: ([normal((4, 24, 5, 6), f32, seed=1).to(d).to(memory_format=torch.channels_last), normal((4, 24, 5, 6), f32, seed=2).to(d)], {}), tag="channels_last_plus_nchw")
    add(aten.where.self, lambda d: ([(normal((3, 16, 4, 5), f32, seed=1) > 0).to(d).to(memory_format=torch.channels_last), normal((3, 16, 4, 5), f32, seed=2).to(d).to(memory_format=torch.channels_last), normal((16, 1, 1), f32, seed=3).to(d)], {}), exact=True, tag="channels_last_three_way")

    # ---- unary: relu / clamp
    for dt in (f32, f16, bf16):
        t = f"{dt}".split(".")[-1]
        add(aten.relu.default, lambda d, dt=dt: (_to(d, normal((33, 65), dt, seed=1)), {}), tag=t)
        add(aten.clamp.default, lambda d, dt=dt: (_to(d, normal((33, 65), dt, seed=1), -0.5, 0.75), {}), tag=t)
    for dt in (f32, bf16, torch.float64):   # sign of zero and NaN survive bit for bit
        add(aten.relu.default, lambda d, dt=dt: (_to(d, torch.tensor([-0.0, 0.0, -1.0, float("nan"), float("-inf"), float("inf"), 2.5], dtype=dt)), {}),
            exact=True, tag=f"signed_zero_{str(dt)[6:]}")
    for op, extra in ((aten.relu.default, ()), (aten.clamp.default, (-1, 1))):
        add(op, lambda d, extra=extra: ([special(f32).to(d), *extra], {}), tag="special")
        add(op, lambda d, extra=extra: ([poison(normal((40, 24), f16, seed=2), 0.05, 3).to(d).t(), *extra], {}), tag="naninf_t")
        add(op, lambda d, extra=extra: ([normal((16, 64), f32, seed=5).to(d)[:, 1::3], *extra], {}), tag="strided")
        add(op, lambda d, extra=extra: ([torch.empty(0, 128, dtype=f16).to(d), *extra], {}), tag="empty")
        add(op, lambda d, extra=extra: ([torch.tensor(-1.5, dtype=f16).to(d), *extra], {}), tag="0d")
        add(op, lambda d, extra=extra: ([randint((30,), 10, 1, i32, -10).to(d), *extra], {}), exact=True, tag="i32")
        add(op, lambda d, extra=extra: ([normal((2, 3, 4, 5), f32, seed=1).to(d).permute(3, 1, 0, 2), *extra], {}), tag="perm4")
    add(aten.clamp.default, lambda d: (_to(d, normal((50,), f32, seed=1), None, 0.25), {}), tag="max_only")
    add(aten.clamp.default, lambda d: (_to(d, normal((50,), f32, seed=1), 0.25), {}), tag="min_only")
    add(aten.clamp.default, lambda d: (_to(d, normal((50,), f32, seed=1), 2, 1), {}), tag="lo_gt_hi")
    add(aten.clamp.default, lambda d: (_to(d, normal((50,), f32, seed=1), float("nan"), 1.0), {}), tag="nan_bound")
    add(aten.clamp.default, lambda d: (_to(d, randint((50,), 10, 1, i32, -10), 0.5, 2), {}), tag="int_float_bounds")
    add(aten.clamp.default, lambda d: (_to(d, normal((50,), bf16, seed=1), -0.3, 0.3), {}), tag="bf16_inexact_bounds")

    for op, b in ((aten.clamp_min.default, -0.25), (aten.clamp_max.default, 0.5)):
        add(op, lambda d, b=b: (_to(d, poison(normal((33, 65), f32, seed=1), 0.05, 2), b), {}), tag="f32_naninf")
        add(op, lambda d, b=b: ([normal((40, 24), bf16, seed=2).to(d).t(), b], {}), tag="bf16_t")
        add(op, lambda d, b=b: (_to(d, randint((30,), 10, 1, i32, -10), 2), {}), exact=True, tag="i32")
        add(op, lambda d, b=b: (_to(d, torch.empty(0, 128, dtype=f16), b), {}), tag="empty")
    add(aten.clamp.Tensor, lambda d: (_to(d, poison(normal((33, 65), f32, seed=1), 0.05, 2), normal((33, 65), f32, -1, 0.2, seed=3), normal((33, 65), f32, 1, 0.2, seed=4)), {}), tag="both")
    add(aten.clamp.Tensor, lambda d: (_to(d, normal((6, 40), f16, seed=1), normal((40,), f16, -0.5, 0.1, seed=3), None), {}), tag="min_bcast")
    add(aten.clamp.Tensor, lambda d: (_to(d, normal((6, 40), bf16, seed=1), None, torch.tensor(0.25, dtype=bf16)), {}), tag="max_0d")
    add(aten.clamp.Tensor, lambda d: (_to(d, normal((50,), f32, seed=1), torch.full((50,), float("nan")), normal((50,), f32, 1, 0.1, seed=2)), {}), tag="nan_bound")

    # ---- where
    cond = lambda shape, seed: normal(shape, f32, seed=seed) > 0
    for dt in (f32, f16, bf16, i64):
        mk = (lambda s, sd, dt=dt: randint(s, 100, sd, dt, -100)) if dt == i64 else (lambda s, sd, dt=dt: poison(normal(s, dt, seed=sd), 0.05, sd))
        add(aten.where.self, lambda d, mk=mk: (_to(d, cond((33, 65), 1), mk((33, 65), 2), mk((33, 65), 3)), {}), exact=True, tag=f"{dt}".split(".")[-1])
    add(aten.where.self, lambda d: (_to(d, cond((4, 1, 16), 1), normal((1, 5, 16), f16, seed=2), normal((4, 5, 1), f16, seed=3)), {}), exact=True, tag="bcast3")
    add(aten.where.self, lambda d: ([cond((48, 20), 1).to(d).t(), normal((48, 20), f16, seed=2).to(d).t(), normal((48, 20), f16, seed=3).to(d).t()], {}), exact=True, tag="all_t")
    add(aten.where.self, lambda d: ([cond((20, 48), 1).to(d), normal((48, 20), f16, seed=2).to(d).t(), normal((20, 48), f16, seed=3).to(d)], {}), exact=True, tag="mixed_layout")
    add(aten.where.self, lambda d: (_to(d, cond((9,), 1), normal((9,), f16, seed=2), normal((9,), f32, seed=3)), {}), tag="promote")
    add(aten.where.self, lambda d: (_to(d, cond((0, 128), 1), torch.empty(0, 128, dtype=f16), torch.empty(0, 128, dtype=f16)), {}), exact=True, tag="empty")
    add(aten.where.self, lambda d: (_to(d, torch.tensor(True), torch.tensor(1.0), torch.tensor(2.0)), {}), exact=True, tag="0d")
    add(aten.where.self, lambda d: (_to(d, cond((6, 7), 1), normal((6, 7), f32, seed=2), torch.tensor(0.0)), {}), exact=True, tag="0d_other")

    # ---- reductions: sum / mean / amax / argmax
    def red_variants(op, has_dtype, needs_list, allow_int=True, argmax=False):
        def dims(v):
            if argmax:
                return v if not isinstance(v, list) else v[0]
            return v if not needs_list or isinstance(v, list) else [v]
        ex = argmax
        for dt in (f32, f16, bf16):
            t = f"{dt}".split(".")[-1]
            add(op, lambda d, dt=dt: (_to(d, normal((37, 129), dt, seed=1), dims(-1)), {}), exact=ex, tag=f"last_{t}")
            add(op, lambda d, dt=dt: (_to(d, normal((37, 129), dt, seed=1), dims(0)), {}), exact=ex, tag=f"first_{t}")
        add(op, lambda d: (_to(d, normal((5, 300, 7), f32, seed=1), dims(1), True), {}), exact=ex, tag="mid_keepdim")
        add(op, lambda d: (_to(d, normal((64, 4096), bf16, 0, 2, seed=1), dims(-1)), {}), exact=ex, tag="row4096")
        add(op, lambda d: (_to(d, normal((3, 70001), f32, seed=1), dims(-1)), {}), exact=ex, tag="long_rows")
        add(op, lambda d: (_to(d, normal((5000, 6), f32, seed=1), dims(-1)), {}), exact=ex, tag="short_rows")
        add(op, lambda d: (_to(d, normal((2, 400000), f32, seed=1), dims(-1)), {}), exact=ex, tag="split_rows")
        add(op, lambda d: (_to(d, normal((3000, 5), f32, seed=1), dims(0)), {}), exact=ex, tag="split_cols")
        add(op, lambda d: ([normal((40, 24), f32, seed=2).to(d).t(), dims(-1)], {}), exact=ex, tag="transposed")
        add(op, lambda d: (_to(d, torch.tensor(2.5, dtype=f32), *(() if argmax else (dims([]),))), {}), exact=ex, tag="0d")
        if not argmax:
            add(op, lambda d: (_to(d, normal((4, 5, 6), f32, seed=1), [0, 2]), {}), tag="dims_0_2")
            add(op, lambda d: (_to(d, normal((4, 5, 6), f32, seed=1), [1, 2]), {}), tag="dims_1_2")
            add(op, lambda d: (_to(d, normal((4, 5, 6), f32, seed=1), [-1, 0, 1], True), {}), tag="all_keepdim")
            add(op, lambda d: (_to(d, normal((4, 5, 6), f32, seed=1), []), {}), tag="dim_empty_list")
        add(op, lambda d: (_to(d, torch.empty(0, 128, dtype=f16), dims(-1)), {}), exact=ex, tag="empty_outer")
        if allow_int:
            add(op, lambda d: (_to(d, randint((13, 50), 1000, 1, i32, -1000), dims(-1)), {}), exact=True, tag="i32")
            add(op, lambda d: (_to(d, randint((13, 50), 1000, 1, i64, -1000), dims(0)), {}), exact=True, tag="i64")
        if has_dtype:
            add(op, lambda d: (_to(d, normal((37, 129), bf16, seed=1), dims(-1)), {"dtype": f32}), tag="dtype_f32")
            add(op, lambda d: (_to(d, normal((37, 129), f32, seed=1), dims(-1)), {"dtype": bf16}), tag="dtype_bf16")

    red_variants(aten.sum.dim_IntList, True, True)
    red_variants(aten.mean.dim, True, True, allow_int=False)
    red_variants(aten.amax.default, False, True)
    red_variants(aten.argmax.default, False, False, argmax=True)
    add(aten.sum.dim_IntList, lambda d: (_to(d, torch.empty(128, 0, dtype=f32), [-1]), {}), tag="empty_reduced")
    add(aten.mean.dim, lambda d: (_to(d, torch.empty(4, 0, dtype=f32), [-1]), {}), tag="empty_reduced_nan")
    add(aten.sum.dim_IntList, lambda d: (_to(d, normal((20, 30), f32, seed=1) > 0, [-1]), {}), exact=True, tag="bool")
    add(aten.sum.dim_IntList, lambda d: (_to(d, normal((20, 30), f32, seed=1), None), {}), tag="dim_none")
    add(aten.sum.default, lambda d: (_to(d, normal((300, 500), f32, seed=1)), {}), tag="all")
    add(aten.sum.default, lambda d: (_to(d, normal((300, 500), bf16, seed=1)), {"dtype": f32}), tag="all_dtype")
    add(aten.sum.default, lambda d: (_to(d, randint((300, 50), 10, 1, i32)), {}), exact=True, tag="all_int")
    add(aten.mean.default, lambda d: (_to(d, normal((300, 500), f32, 3.0, 1.0, seed=1)), {}), tag="all")
    add(aten.mean.default, lambda d: (_to(d, normal((30, 50), f16, seed=1)), {}), tag="all_f16")
    nan_rows = lambda dt: torch.tensor([[1, float("nan"), 5, 5], [2, 7, 7, float("-inf")], [float("inf"), 1, float("inf"), 0],
                                        [float("-inf")] * 4, [float("nan")] * 4], dtype=dt)
    for dt in (f32, bf16):
        t = f"{dt}".split(".")[-1]
        add(aten.amax.default, lambda d, dt=dt: (_to(d, nan_rows(dt), [-1]), {}), tag=f"nan_ties_{t}")
        add(aten.argmax.default, lambda d, dt=dt: (_to(d, nan_rows(dt), -1), {}), exact=True, tag=f"nan_ties_{t}")
        add(aten.argmax.default, lambda d, dt=dt: (_to(d, nan_rows(dt), 0), {}), exact=True, tag=f"nan_ties_dim0_{t}")
        add(aten.sum.dim_IntList, lambda d, dt=dt: (_to(d, nan_rows(dt), [-1]), {}), tag=f"nan_{t}")
    add(aten.argmax.default, lambda d: (_to(d, normal((37, 129), f32, seed=1)), {}), exact=True, tag="flat")
    add(aten.argmax.default, lambda d: (_to(d, normal((37, 129), f32, seed=1), None, True), {}), exact=True, tag="flat_keepdim")
    add(aten.argmax.default, lambda d: (_to(d, normal((5, 300, 7), f32, seed=1), 1, True), {}), exact=True, tag="mid_keepdim2")
    add(aten.argmax.default, lambda d: (_to(d, torch.zeros(6, 5000, dtype=f32), -1), {}), exact=True, tag="all_ties")
    add(aten.argmax.default, lambda d: (_to(d, (normal((16, 70000), f32, seed=2) * 4).round(), -1), {}), exact=True, tag="many_ties")
    # many short rows (global average pooling over a 7x7 map): sixteen lanes per row, scalar and
    # vector forms, a row count that is not a multiple of the four rows a wave holds
    for red, dt in ((9, f32), (16, f32), (33, bf16), (49, f16), (64, f32), (100, bf16), (128, f16)):
        t = f"{dt}".split(".")[-1]
        rows = 8192 + 5
        add(aten.sum.dim_IntList, lambda d, red=red, dt=dt, rows=rows: (_to(d, normal((rows, red), dt, seed=1), [-1]), {}), tag=f"short_rows_{red}_{t}")
        add(aten.mean.dim, lambda d, red=red, dt=dt, rows=rows: (_to(d, normal((rows, red), dt, 3.0, seed=2), [-1], True), {}), tag=f"short_rows_{red}_{t}")
        add(aten.amax.default, lambda d, red=red, dt=dt, rows=rows: (_to(d, poison(normal((rows, red), dt, seed=3), 0.002, 5), [-1]), {}), tag=f"short_rows_{red}_{t}")
        add(aten.argmax.default, lambda d, red=red, dt=dt, rows=rows: (_to(d, poison((normal((rows, red), dt, seed=4) * 2).round(), 0.002, 6), -1), {}), exact=True, tag=f"short_rows_{red}_{t}")
    add(aten.mean.dim, lambda d: (_to(d, normal((16, 600, 7, 7), f16, 1.0, seed=1), [-1, -2], True), {}), tag="pool_7x7")
    # many misaligned rows of 129 .. 512 elements (a 197-wide attention row): sixteen lanes per row over the aligned window
    for red, dt in ((197, f16), (131, f32), (255, bf16), (509, f16)):
        t = f"{dt}".split(".")[-1]
        add(aten.sum.dim_IntList, lambda d, red=red, dt=dt: (_to(d, normal((8200, red), dt, seed=1), [-1], True), {}), tag=f"attn_rows_{red}_{t}")
        add(aten.amax.default, lambda d, red=red, dt=dt: (_to(d, poison(normal((8200, red), dt, seed=3), 0.002, 5), [-1]), {}), tag=f"attn_rows_{red}_{t}")
        add(aten.argmax.default, lambda d, red=red, dt=dt: (_to(d, poison((normal((8200, red), dt, seed=4) * 2).round(), 0.002, 6), -1), {}), exact=True, tag=f"attn_rows_{red}_{t}")
    add(aten.sum.dim_IntList, lambda d: (_to(d, randint((9000, 40), 100, 1, i32, low=-100), [-1]), {}), exact=True, tag="short_rows_int")
    add(aten.sum.dim_IntList, lambda d: ([normal((9000 * 64 + 1,), f32, seed=7).to(d)[1:].view(9000, 64), [-1]], {}), tag="short_rows_offset_view")

    # a long reduced axis over few columns: transposed to rows first
    add(aten.sum.dim_IntList, lambda d: (_to(d, normal((70000, 8), f16, 0, 1, seed=1), [0]), {}), tag="few_columns_f16")
    add(aten.amax.default, lambda d: (_to(d, poison(normal((3000, 50), f32, seed=1), 0.0001, 4), [0]), {}), tag="few_columns_naninf")
    add(aten.argmax.default, lambda d: (_to(d, torch.round(normal((4, 9000, 5), f32, 0, 3, seed=1)), 1), {}), exact=True, tag="few_columns_ties")
    add(aten.mean.dim, lambda d: (_to(d, normal((2, 5000, 16), bf16, 1, 2, seed=1), [1], True), {}), tag="few_columns_keepdim_bf16")
    add(aten.sum.dim_IntList, lambda d: ([normal((70000, 8), f32, 0, 1, seed=1).to(d).t(), [1]], {}), tag="few_columns_transposed_view")
    add(aten.sum.dim_IntList, lambda d: (_to(d, randint((40000, 6), 100, 1, i32), [0]), {}), exact=True, tag="few_columns_int")
    # ---- _softmax
    for dt in (f32, f16, bf16):
        t = f"{dt}".split(".")[-1]
        add(aten._softmax.default, lambda d, dt=dt: (_to(d, normal((37, 129), dt, 0, 2, seed=1), -1, False), {}), tag=f"last_{t}")
        add(aten._softmax.default, lambda d, dt=dt: (_to(d, normal((37, 129), dt, 0, 2, seed=1), 0, False), {}), tag=f"first_{t}")
    add(aten._softmax.default, lambda d: (_to(d, normal((16, 4096), bf16, 0, 2, seed=1), -1, False), {}), tag="row4096")
    add(aten._softmax.default, lambda d: (_to(d, normal((4, 8192), f32, 0, 2, seed=1), 1, False), {}), tag="row8192_f32")
    add(aten._softmax.default, lambda d: (_to(d, normal((3, 50000), f32, 0, 2, seed=1), -1, False), {}), tag="long_rows")
    add(aten._softmax.default, lambda d: (_to(d, normal((3, 20000), bf16, 0, 2, seed=1), -1, False), {}), tag="long_rows_bf16")
    add(aten._softmax.default, lambda d: (_to(d, normal((5, 300, 7), f32, seed=1), 1, False), {}), tag="mid")
    add(aten._log_softmax.default, lambda d: (_to(d, poison(normal((3, 100, 33), f16, 0, 2, seed=1), 0.002, 4), 1, False), {}), tag="mid_odd_inner_f16")
    add(aten._softmax.default, lambda d: (_to(d, normal((2, 40, 49), bf16, 0, 2, seed=1), 1, False), {}), tag="mid_7x7_bf16")
    add(aten._softmax.default, lambda d: (_to(d, normal((64, 520), f32, 0, 2, seed=1), 0, False), {}), tag="first_dim_few_blocks")
    add(aten._softmax.default, lambda d: ([normal((40, 24), f32, seed=2).to(d).t(), -1, False], {}), tag="transposed")
    add(aten._softmax.default, lambda d: (_to(d, torch.tensor([[float("-inf"), float("-inf")], [float("inf"), 1.0], [float("nan"), 1.0],
                                                                 [float("-inf"), 0.0], [1.0, 2.0]], dtype=f32), -1, False), {}), tag="special")
    add(aten._softmax.default, lambda d: (_to(d, torch.cat([torch.full((2, 9000), float("-inf")), normal((2, 9000), f32, seed=1)], 0), -1, False), {}), tag="special_long")
    add(aten._softmax.default, lambda d: (_to(d, torch.empty(0, 128, dtype=f16), -1, False), {}), tag="empty")
    add(aten._softmax.default, lambda d: (_to(d, torch.tensor(0.3, dtype=f32), 0, False), {}), tag="0d")
    add(aten._softmax.default, lambda d: (_to(d, normal((37, 129), bf16, 0, 2, seed=1), -1, True), {}), tag="half_to_float", stock_gpu=False)

    for dt in (f32, f16, bf16):
        t = f"{dt}".split(".")[-1]
        add(aten._log_softmax.default, lambda d, dt=dt: (_to(d, normal((37, 129), dt, 0, 2, seed=1), -1, False), {}), tag=f"last_{t}")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((16, 4096), bf16, 0, 2, seed=1), -1, False), {}), tag="row4096")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((3, 50000), f32, 0, 2, seed=1), -1, False), {}), tag="long_rows")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((5, 300, 7), f32, seed=1), 1, False), {}), tag="mid")
    add(aten._log_softmax.default, lambda d: (_to(d, torch.tensor([[float("-inf"), float("-inf")], [float("inf"), 1.0], [float("nan"), 1.0],
                                                                     [float("-inf"), 0.0], [1.0, 2.0]], dtype=f32), -1, False), {}), tag="special")
    add(aten._log_softmax.default, lambda d: (_to(d, torch.empty(0, 128, dtype=f16), -1, False), {}), tag="empty")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((37, 129), bf16, 0, 2, seed=1), -1, True), {}), tag="half_to_float", stock_gpu=False)

    # softmax axis is not the last one, inner extent a multiple of the vector width
    add(aten._softmax.default, lambda d: (_to(d, normal((4, 100, 64), f16, 0, 2, seed=1), 1, False), {}), tag="mid_vec_f16")
    add(aten._softmax.default, lambda d: (_to(d, normal((3, 40, 8, 16), f32, 0, 2, seed=1), 1, False), {}), tag="mid_vec_f32")
    add(aten._softmax.default, lambda d: (_to(d, normal((64, 256), bf16, 0, 2, seed=1), 0, True), {}), tag="dim0_half_to_float", stock_gpu=False)
    add(aten._log_softmax.default, lambda d: (_to(d, poison(normal((2, 33, 520), f16, 0, 2, seed=1), 0.01, 4), 1, False), {}), tag="mid_vec_naninf")
    # odd row lengths: rows start off 16-byte boundaries (shifted vector access, all row tile widths)
    add(aten._softmax.default, lambda d: (_to(d, normal((300, 2049), f16, 0, 2, seed=1), -1, False), {}), tag="odd_2049_f16")
    add(aten._softmax.default, lambda d: (_to(d, normal((33, 1001), f32, 0, 2, seed=1), -1, False), {}), tag="odd_1001_f32")
    add(aten._softmax.default, lambda d: (_to(d, normal((64, 197), f16, 0, 2, seed=1), -1, True), {}), tag="odd_197_half_to_float")
    add(aten._softmax.default, lambda d: (_to(d, normal((9, 16385), bf16, 0, 2, seed=1), -1, False), {}), tag="odd_16385_bf16")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((5, 50257), f16, 0, 2, seed=1), -1, False), {}), tag="odd_50257_f16")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((3, 40001), f32, 0, 2, seed=1), -1, False), {}), tag="odd_40001_f32")
    f64 = torch.float64
    add(aten._softmax.default, lambda d: (_to(d, normal((37, 129), f64, 0, 2, seed=1), -1, False), {}), tag="last_f64")
    add(aten._softmax.default, lambda d: (_to(d, normal((5, 30, 7), f64, seed=1), 1, False), {}), tag="mid_f64")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((3, 5000), f64, 0, 2, seed=1), -1, False), {}), tag="long_rows_f64")
    # softmax axis in the middle with a short inner extent: transposed to rows and back
    add(aten._softmax.default, lambda d: (_to(d, normal((8, 400, 49), f32, 0, 2, seed=1), 1, False), {}), tag="mid_short_inner_f32")
    add(aten._log_softmax.default, lambda d: (_to(d, poison(normal((4, 300, 60), bf16, 0, 2, seed=1), 0.002, 4), 1, False), {}), tag="mid_short_inner_naninf_bf16")
    add(aten._softmax.default, lambda d: (_to(d, normal((12, 256, 48), f16, 0, 2, seed=1), 1, True), {}), tag="mid_short_inner_half_to_float")
    add(aten._softmax.default, lambda d: (_to(d, normal((2100, 8, 8), f32, 0, 2, seed=1), 0, False), {}), tag="first_dim_8x8_inner")
    # short rows: 1, 2, 4, 8, 16 and 32 lanes per row, vector and single-element layouts
    for rl, dt, t in ((2, f32, "f32"), (3, f16, "f16"), (8, f32, "f32"), (10, f32, "f32"), (16, bf16, "bf16"), (24, f16, "f16"),
                     (49, f32, "f32"), (64, f16, "f16"), (100, bf16, "bf16"), (128, f32, "f32"), (255, f16, "f16"), (256, bf16, "bf16")):
        add(aten._softmax.default, lambda d, rl=rl, dt=dt: (_to(d, normal((1037, rl), dt, 0, 2, seed=rl), -1, False), {}), tag=f"short_{rl}_{t}")
    add(aten._log_softmax.default, lambda d: (_to(d, poison(normal((515, 8), f32, 0, 2, seed=1), 0.01, 4), -1, False), {}), tag="short_8_naninf")
    add(aten._log_softmax.default, lambda d: (_to(d, poison(normal((130, 40), f16, 0, 2, seed=1), 0.005, 4), -1, False), {}), tag="short_40_naninf_f16")
    add(aten._softmax.default, lambda d: (_to(d, normal((333, 64), f16, 0, 2, seed=1), -1, True), {}), tag="short_64_half_to_float")
    add(aten._log_softmax.default, lambda d: (_to(d, normal((77, 10), bf16, 0, 2, seed=1), -1, True), {}), tag="short_10_half_to_float", stock_gpu=False)
    add(aten._softmax.default, lambda d: ([normal((64, 40), f32, 0, 2, seed=1).to(d)[:, 4:36], -1, False], {}), tag="short_row_slice")
    # short rows: 1 .. 32 lanes per row, vector and single-element layouts, every gamma / beta combination
    for rl, dt, t, hw, hb in ((4, f32, "f32", True, True), (8, f16, "f16", True, False), (10, f32, "f32", True, True), (16, bf16, "bf16", False, True),
                              (49, f32, "f32", True, True), (64, f16, "f16", True, True), (100, bf16, "bf16", False, False), (128, f32, "f32", True, True),
                              (128, bf16, "bf16", True, True), (255, f16, "f16", True, True), (256, bf16, "bf16", True, False)):
        add(aten.native_layer_norm.default,
            lambda d, rl=rl, dt=dt, hw=hw, hb=hb: (_to(d, normal((1037, rl), dt, 1, 2, seed=rl), [rl], normal((rl,), dt, 1, 0.1, seed=2) if hw else None,
                                                      normal((rl,), dt, 0, 0.1, seed=3) if hb else None, 1e-5), {}), tag=f"short_{rl}_{t}")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((300, 12, 64), f16, 0, 2, seed=1), [64], normal((64,), f32, 1, 0.1, seed=2), normal((64,), f32, 0, 0.1, seed=3), 1e-6), {}), tag="short_64_f32_params", stock_gpu=False)
    # a thousand and more mid-length rows: the streaming kernels (one wave per row, next row prefetched), four- and
    # eight-slab register tiles, rows that do not fill the last slab, row counts that do not divide by the waves
    for rows, rl, dt, t, hw, hb in ((1100, 1000, f32, "f32", True, True), (1030, 1800, f32, "f32", True, False), (1500, 2056, bf16, "bf16", False, False),
                                    (1024, 4096, f16, "f16", True, True), (2050, 520, bf16, "bf16", False, True), (1027, 2048, f32, "f32", True, True)):
        add(aten.native_layer_norm.default,
            lambda d, rows=rows, rl=rl, dt=dt, hw=hw, hb=hb: (_to(d, normal((rows, rl), dt, 1, 2, seed=rl), [rl], normal((rl,), dt, 1, 0.1, seed=2) if hw else None,
                                                                 normal((rl,), dt, 0, 0.1, seed=3) if hb else None, 1e-5), {}), tag=f"stream_{rows}x{rl}_{t}")
        add(aten._softmax.default if hw else aten._log_softmax.default,
            lambda d, rows=rows, rl=rl, dt=dt: (_to(d, poison(normal((rows, rl), dt, 0, 2, seed=rl + 1), 0.0002, 5), -1, False), {}), tag=f"stream_{rows}x{rl}_{t}")
    # long rows: 8- and 16-wave register tiles, then the two-pass block kernel
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((5, 12288), bf16, 1, 2, seed=1), [12288], normal((12288,), bf16, 1, 0.1, seed=2), normal((12288,), bf16, 0, 0.1, seed=3), 1e-5), {}), tag="row12288_bf16")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((3, 40000), f32, -2, 3, seed=1), [40000], normal((40000,), f32, 1, 0.1, seed=2), None, 1e-5), {}), tag="row40000_f32")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((2, 70000), f16, 0, 1, seed=1), [70000], None, normal((70000,), f16, 0, 0.1, seed=3), 1e-5), {}), tag="row70000_f16")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((33, 300), f64, 3, 2, seed=1), [300], normal((300,), f64, 1, 0.1, seed=2), normal((300,), f64, 0, 0.1, seed=3), 1e-5), {}), tag="f64")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((4, 6, 10), f64, seed=1), [6, 10], None, None, 1e-5), {}), tag="f64_no_affine_2d")

    # ---- native_layer_norm
    for dt in (f32, f16, bf16):
        t = f"{dt}".split(".")[-1]
        add(aten.native_layer_norm.default,
            lambda d, dt=dt: (_to(d, normal((37, 129), dt, 0, 2, seed=1), [129], normal((129,), dt, 1, 0.1, seed=2), normal((129,), dt, 0, 0.1, seed=3), 1e-5), {}), tag=t)
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((16, 4096), bf16, 0, 2, seed=1), [4096], normal((4096,), bf16, 1, 0.1, seed=2), normal((4096,), bf16, 0, 0.1, seed=3), 1e-5), {}), tag="row4096")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((16, 4096), bf16, 0, 2, seed=1), [4096], normal((4096,), f32, 1, 0.1, seed=2), normal((4096,), f32, 0, 0.1, seed=3), 1e-5), {}), tag="f32_params", stock_gpu=False)
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((3, 30000), f32, 5.0, 2, seed=1), [30000], normal((30000,), f32, 1, 0.1, seed=2), normal((30000,), f32, 0, 0.1, seed=3), 1e-5), {}), tag="long_rows")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((2, 3, 4, 5), f32, seed=1), [4, 5], normal((4, 5), f32, 1, 0.1, seed=2), normal((4, 5), f32, 0, 0.1, seed=3), 1e-5), {}), tag="multi_dim")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((37, 129), f32, seed=1), [129], None, None, 1e-5), {}), tag="no_affine")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((37, 129), f32, seed=1), [129], normal((129,), f32, 1, 0.1, seed=2), None, 1e-3), {}), tag="weight_only")
    add(aten.native_layer_norm.default, lambda d: (_to(d, torch.empty(0, 8, dtype=f32), [8], normal((8,), f32, seed=2), normal((8,), f32, seed=3), 1e-5), {}), tag="empty")
    add(aten.native_layer_norm.default, lambda d: ([normal((24, 40), f32, seed=2).to(d).t(), [24], None, None, 1e-5], {}), tag="transposed")
    add(aten.native_layer_norm.default, lambda d: (_to(d, normal((64, 1024), f32, 1000.0, 0.5, seed=1), [1024], None, None, 1e-5), {}), tag="large_mean")

    # ---- mm / addmm
    for dt in (bf16, f16, f32):
        t = f"{dt}".split(".")[-1]
        add(aten.mm.default, lambda d, dt=dt: (_to(d, normal((256, 128), dt, seed=1), normal((128, 512), dt, 0, 0.1, seed=2)), {}), tag=f"tile_{t}")
        add(aten.mm.default, lambda d, dt=dt: (_to(d, normal((37, 53), dt, seed=1), normal((53, 29), dt, 0, 0.1, seed=2)), {}), tag=f"ragged_{t}")
        add(aten.addmm.default, lambda d, dt=dt: (_to(d, normal((512,), dt, seed=3), normal((256, 128), dt, seed=1), normal((128, 512), dt, 0, 0.1, seed=2)), {}), tag=f"bias_{t}")
    add(aten.mm.default, lambda d: (_to(d, normal((300, 264), bf16, seed=1), normal((264, 520), bf16, 0, 0.1, seed=2)), {}), tag="edge_tiles")
    add(aten.mm.default, lambda d: (_to(d, normal((512, 1024), bf16, seed=1), normal((1024, 768), bf16, 0, 0.05, seed=2)), {}), tag="multi_tile")
    for k in (32, 64, 96, 128, 192, 320, 448):   # every prologue / steady-state / drain length of the K loops
        add(aten.mm.default, lambda d, k=k: (_to(d, normal((260, k), bf16, seed=1), normal((k, 264), bf16, 0, 0.1, seed=2)), {}), tag=f"ksteps_{k}")
    add(aten.mm.default, lambda d: ([normal((512, 320), bf16, seed=1).to(d), normal((768, 320), bf16, 0, 0.05, seed=2).to(d).t()], {}), tag="b_transposed")
    for k in (16, 32, 48, 64, 80, 272):   # fp32 MFMA path: every prologue / steady-state / drain length
        add(aten.mm.default, lambda d, k=k: (_to(d, normal((132, k), f32, seed=1), normal((k, 140), f32, 0, 0.1, seed=2)), {}), tag=f"f32_ksteps_{k}")
    add(aten.mm.default, lambda d: ([normal((300, 96), f32, seed=1).to(d), normal((260, 96), f32, 0, 0.1, seed=2).to(d).t()], {}), tag="f32_b_transposed")
    # more 128x128 tiles than CUs: the four-stage fp32 ring, two workgroups per CU (fewer tiles take the eight-stage ring)
    # 196 tiles of 128x128: one workgroup per CU, the eight-stage ring on the large tiles
    add(aten.mm.default, lambda d: (_to(d, normal((1700, 176), f32, seed=1), normal((176, 1752), f32, 0, 0.1, seed=2)), {}), tag="f32_196_tiles_k176")
    add(aten.addmm.default, lambda d: ([normal((1700, 1), f32, seed=3).to(d), normal((1700, 80), f32, seed=1).to(d), normal((1750, 80), f32, 0, 0.1, seed=2).to(d).t()], {}), tag="f32_196_tiles_k80_nt_col_bias")
    add(aten.mm.default, lambda d: (_to(d, normal((2100, 48), f32, seed=1), normal((48, 2064), f32, 0, 0.1, seed=2)), {}), tag="f32_many_tiles_k48")
    add(aten.mm.default, lambda d: ([normal((2100, 208), f32, seed=1).to(d), normal((2064, 208), f32, 0, 0.1, seed=2).to(d).t()], {}), tag="f32_many_tiles_k208_nt")
    add(aten.addmm.default, lambda d: ([normal((260,), f32, seed=3).to(d), normal((300, 96), f32, seed=1).to(d), normal((260, 96), f32, 0, 0.1, seed=2).to(d).t()], {"beta": 0.5, "alpha": 2.0}), tag="f32_linear")
    add(aten.mm.default, lambda d: (_to(d, torch.eye(128, dtype=f32), normal((128, 128), f32, seed=2)), {}), exact=True, tag="f32_identity")
    add(aten.mm.default, lambda d: (_to(d, normal((70, 90), torch.float64, seed=1), normal((90, 50), torch.float64, 0, 0.1, seed=2)), {}), tag="f64")
    add(aten.addmm.default, lambda d: (_to(d, normal((50,), torch.float64, seed=3), normal((70, 90), torch.float64, seed=1), normal((90, 50), torch.float64, 0, 0.1, seed=2)), {"beta": 0.5}), tag="f64")
    add(aten.mm.default, lambda d: ([normal((512, 700), bf16, seed=1).to(d)[:, ::2], normal((350, 264), bf16, 0, 0.05, seed=2).to(d)], {}), tag="a_strided_cols")
    add(aten.mm.default, lambda d: ([normal((256, 320), bf16, seed=1).to(d), normal((320, 600), bf16, 0, 0.05, seed=2).to(d)[:, ::2]], {}), tag="b_strided_cols")
    # output width not a multiple of the vector width (transposed B, e.g. a 50257-wide vocabulary): element stores
    add(aten.mm.default, lambda d: ([normal((300, 96), bf16, seed=1).to(d), normal((261, 96), bf16, 0, 0.1, seed=2).to(d).t()], {}), tag="odd_n_bf16")
    add(aten.mm.default, lambda d: ([normal((300, 96), f32, seed=1).to(d), normal((261, 96), f32, 0, 0.1, seed=2).to(d).t()], {}), tag="odd_n_f32")
    add(aten.addmm.default, lambda d: ([normal((263,), f16, seed=3).to(d), normal((300, 128), f16, seed=1).to(d), normal((263, 128), f16, 0, 0.1, seed=2).to(d).t()], {"beta": 0.5}), tag="odd_n_bias_f16")
    add(aten.addmm.default, lambda d: ([normal((300, 263), f32, seed=3).to(d), normal((300, 128), f32, seed=1).to(d), normal((263, 128), f32, 0, 0.1, seed=2).to(d).t()], {"alpha": 2.0}), tag="odd_n_full_c_f32")
    add(aten.mm.default, lambda d: ([normal((64, 768), f16, seed=1).to(d), normal((50257, 768), f16, 0, 0.05, seed=2).to(d).t()], {}), tag="vocab_50257_f16")
    # skinny problems with a long K: split along K over the chip, fp32 partials, finishing pass
    add(aten.mm.default, lambda d: (_to(d, normal((16, 2048), bf16, seed=1), normal((2048, 1024), bf16, 0, 0.05, seed=2)), {}), tag="splitk_bf16")
    add(aten.mm.default, lambda d: (_to(d, normal((40, 2144), f16, seed=1), normal((2144, 520), f16, 0, 0.05, seed=2)), {}), tag="splitk_ragged_f16")
    add(aten.addmm.default, lambda d: ([normal((1024,), bf16, seed=3).to(d), normal((24, 4096), bf16, seed=1).to(d), normal((1024, 4096), bf16, 0, 0.02, seed=2).to(d).t()], {"beta": 0.5, "alpha": 2.0}), tag="splitk_linear_bf16")
    add(aten.addmm.default, lambda d: ([normal((200,), f32, seed=3).to(d), normal((64, 1024), f32, seed=1).to(d), normal((200, 1024), f32, 0, 0.05, seed=2).to(d).t()], {}), tag="splitk_linear_f32")
    add(aten.mm.default, lambda d: (_to(d, normal((64, 1040), f32, seed=1), normal((1040, 256), f32, 0, 0.05, seed=2)), {}), tag="splitk_f32")
    # split-K with an N that is no multiple of 4: partial planes keep padded rows, output rows are stored element-wise
    add(aten.mm.default, lambda d: ([normal((24, 2048), bf16, seed=1).to(d), normal((1001, 2048), bf16, 0, 0.05, seed=2).to(d).t()], {}), tag="splitk_odd_n_bf16")
    add(aten.mm.default, lambda d: (_to(d, normal((64, 1040), f32, seed=1), normal((1040, 250), f32, 0, 0.05, seed=2)), {}), tag="splitk_n250_f32")
    add(aten.addmm.default, lambda d: ([normal((1001,), f16, seed=3).to(d), normal((40, 4096), f16, seed=1).to(d), normal((1001, 4096), f16, 0, 0.02, seed=2).to(d).t()], {"beta": 0.5, "alpha": 2.0}), tag="splitk_odd_n_bias_f16")
    add(aten.mm.default, lambda d: ([normal((320, 512), bf16, seed=1).to(d).t(), normal((320, 768), bf16, 0, 0.05, seed=2).to(d)], {}), tag="a_transposed")
    # layouts the MFMA kernels cannot address directly: K no multiple of the vector (operands copied into zero-padded
    # K-contiguous buffers), a row-major right operand with misaligned rows (re-laid K-contiguous)
    add(aten.mm.default, lambda d: (_to(d, normal((260, 100), bf16, seed=1), normal((100, 264), bf16, 0, 0.1, seed=2)), {}), tag="k_unaligned_bf16")
    add(aten.addmm.default, lambda d: (_to(d, normal((264,), f32, seed=3), normal((130, 50), f32, seed=1), normal((50, 264), f32, 0, 0.1, seed=2)), {"beta": 0.5}), tag="k_unaligned_f32")
    add(aten.mm.default, lambda d: ([poison(normal((300, 37), f16, seed=1), 0.01, 3).to(d), normal((261, 37), f16, 0, 0.1, seed=2).to(d).t()], {}), tag="k_unaligned_specials_f16")
    add(aten.mm.default, lambda d: (_to(d, normal((300, 64), bf16, seed=1), normal((64, 263), bf16, 0, 0.1, seed=2)), {}), tag="nn_odd_n_bf16")
    add(aten.addmm.default, lambda d: (_to(d, normal((1001,), f32, seed=3), normal((70, 128), f32, seed=1), normal((128, 1001), f32, 0, 0.1, seed=2)), {}), tag="nn_odd_n_f32")
    # one row against a large weight (decoding one token): MFMA tiles split along K, not the FMA fallback
    add(aten.mm.default, lambda d: ([normal((1, 2048), bf16, seed=1).to(d), normal((1024, 2048), bf16, 0, 0.05, seed=2).to(d).t()], {}), tag="single_row_bf16")
    add(aten.mm.default, lambda d: (_to(d, normal((1, 4096), f32, seed=1), normal((4096, 1000), f32, 0, 0.05, seed=2)), {}), tag="single_row_f32")
    add(aten.addmm.default, lambda d: ([normal((1024,), f16, seed=3).to(d), normal((3, 2048), f16, seed=1).to(d), normal((1024, 2048), f16, 0, 0.05, seed=2).to(d).t()], {}), tag="three_rows_bias_f16")
    add(aten.mm.default, lambda d: ([normal((2048, 512), bf16, seed=1).to(d).t(), normal((2048, 768), bf16, 0, 0.05, seed=2).to(d)], {}), tag="a_transposed_k2048")
    add(aten.mm.default, lambda d: (_to(d, torch.eye(256, dtype=bf16), normal((256, 256), bf16, seed=2)), {}), exact=True, tag="identity")
    # tiny outputs: long K goes to the MFMA kernels (split along K), the rest to the pipelined generic kernel in every layout
    add(aten.mm.default, lambda d: (_to(d, normal((8, 1024), f16, seed=1), normal((1024, 8), f16, 0, 0.05, seed=2)), {}), tag="tiny_8x8_k1024_f16")
    add(aten.mm.default, lambda d: ([normal((32, 512), bf16, seed=1).to(d), normal((32, 512), bf16, 0, 0.05, seed=2).to(d).t()], {}), tag="tiny_32x32_k512_nt_bf16")
    add(aten.mm.default, lambda d: (_to(d, normal((64, 64), f16, seed=1), normal((64, 64), f16, 0, 0.1, seed=2)), {}), tag="tiny_64_cubed_f16")
    add(aten.mm.default, lambda d: (_to(d, normal((16, 256), f32, seed=1), normal((256, 16), f32, 0, 0.1, seed=2)), {}), tag="tiny_16x16_k256_f32")
    add(aten.mm.default, lambda d: (_to(d, normal((5, 300), f32, seed=1), normal((300, 7), f32, 0, 0.1, seed=2)), {}), tag="tiny_ragged_k300_f32")
    add(aten.mm.default, lambda d: (_to(d, normal((1, 4096), f16, seed=1), normal((4096, 1), f16, 0, 0.02, seed=2)), {}), tag="dot_product_f16")
    add(aten.mm.default, lambda d: (_to(d, normal((2050, 70), f64, seed=1), normal((70, 2041), f64, 0, 0.1, seed=2)), {}), tag="f64_128x128_tiles")
    add(aten.addmm.default, lambda d: ([normal((2041,), f64, seed=3).to(d), normal((70, 2050), f64, seed=1).to(d).t(), normal((2041, 70), f64, 0, 0.1, seed=2).to(d).t()], {"beta": 0.5}), tag="f64_128x128_tiles_both_transposed")
    add(aten.mm.default, lambda d: ([normal((130, 70), f64, seed=1).to(d).t(), normal((50, 130), f64, 0, 0.1, seed=2).to(d).t()], {}), tag="f64_both_transposed")
    add(aten.mm.default, lambda d: ([normal((90, 97), f64, seed=1).to(d), normal((75, 97), f64, 0, 0.1, seed=2).to(d).t()], {}), tag="f64_b_transposed_k97")
    add(aten.addmm.default, lambda d: (_to(d, normal((24,), f16, seed=3), normal((24, 512), f16, seed=1), normal((512, 24), f16, 0, 0.05, seed=2)), {"beta": 0.5, "alpha": 2.0}), tag="tiny_24x24_k512_f16")
    add(aten.mm.default, lambda d: (_to(d, torch.empty(2, 0, dtype=f32), torch.empty(0, 3, dtype=f32)), {}), tag="k0")
    add(aten.mm.default, lambda d: (_to(d, torch.empty(0, 8, dtype=bf16), normal((8, 16), bf16, seed=1)), {}), tag="m0")
    add(aten.addmm.default, lambda d: (_to(d, normal((256, 512), bf16, seed=3), normal((256, 128), bf16, seed=1), normal((128, 512), bf16, 0, 0.1, seed=2)), {"beta": 0.5, "alpha": 2.0}), tag="full_c_alpha_beta")
    add(aten.addmm.default, lambda d: (_to(d, torch.full((512,), float("nan"), dtype=bf16), normal((256, 128), bf16, seed=1), normal((128, 512), bf16, 0, 0.1, seed=2)), {"beta": 0}), tag="beta0_nan")
    add(aten.addmm.default, lambda d: (_to(d, normal((256, 1), f32, seed=3), normal((256, 64), f32, seed=1), normal((64, 40), f32, 0, 0.1, seed=2)), {}), tag="col_bias_f32")
    add(aten.addmm.default, lambda d: (_to(d, normal((29,), f16, seed=3), normal((37, 53), f16, seed=1), normal((53, 29), f16, 0, 0.1, seed=2)), {"alpha": 0.5}), tag="ragged_f16")

    # ---- index_select / embedding / gather
    for dt in (bf16, f32, i64, torch.uint8):
        t = f"{dt}".split(".")[-1]
        src = (lambda s, dt=dt: randint(s, 200, 1, dt)) if not dt.is_floating_point else (lambda s, dt=dt: poison(normal(s, dt, seed=1), 0.02, 2))
        add(aten.index_select.default, lambda d, src=src: (_to(d, src((50, 64)), 0, randint((33,), 50, 3)), {}), exact=True, tag=f"dim0_{t}")
        add(aten.index_select.default, lambda d, src=src: (_to(d, src((7, 50, 9)), 1, randint((33,), 50, 3)), {}), exact=True, tag=f"dim1_{t}")
        add(aten.index_select.default, lambda d, src=src: (_to(d, src((7, 50)), -1, randint((33,), 50, 3, i32)), {}), exact=True, tag=f"last_i32_{t}")
        add(aten.embedding.default, lambda d, src=src: (_to(d, src((50, 64)), randint((4, 5), 50, 3)), {}), exact=True, tag=t)
        add(aten.gather.default, lambda d, src=src: (_to(d, src((20, 64)), 1, randint((20, 64), 64, 3)), {}), exact=True, tag=f"dim1_{t}")
        add(aten.gather.default, lambda d, src=src: (_to(d, src((20, 64)), 0, randint((11, 33), 20, 3)), {}), exact=True, tag=f"dim0_{t}")
    add(aten.index_select.default, lambda d: (_to(d, normal((300, 4096), bf16, seed=1), 0, randint((100,), 300, 3)), {}), exact=True, tag="rows8k")
    for dt, t in ((f16, "f16"), (f32, "f32"), (torch.float64, "f64"), (torch.uint8, "u8")):   # single elements along the last dim: LDS-staged rows
        add(aten.index_select.default, lambda d, dt=dt: ([(normal((37, 1000), f32, 0, 50, seed=1).to(dt)).to(d), -1, randint((300,), 1000, 3).to(d)], {}), exact=True, tag=f"last_lds_{t}")
    add(aten.index_select.default, lambda d: (_to(d, normal((3, 5, 4099), bf16, seed=1), 2, randint((9001,), 4099, 3)), {}), exact=True, tag="last_lds_split")
    add(aten.index_select.default, lambda d: (_to(d, normal((300, 33), bf16, seed=1), 0, randint((100,), 300, 3)), {}), exact=True, tag="odd_row_bytes")
    add(aten.index_select.default, lambda d: ([normal((64, 50), f32, seed=1).to(d).t(), 0, randint((33,), 50, 3).to(d)], {}), exact=True, tag="transposed_src")
    add(aten.index_select.default, lambda d: (_to(d, normal((50, 64), f32, seed=1), 0, torch.tensor(7)), {}), exact=True, tag="0d_index")
    add(aten.index_select.default, lambda d: (_to(d, normal((50, 64), f32, seed=1), 0, torch.empty(0, dtype=i64)), {}), exact=True, tag="empty_index")
    add(aten.index_select.default, lambda d: (_to(d, torch.empty(0, 128, dtype=f16), 1, randint((5,), 128, 3)), {}), exact=True, tag="empty_src")
    add(aten.embedding.default, lambda d: (_to(d, normal((50, 64), bf16, seed=1), torch.tensor(3)), {}), exact=True, tag="0d_index")
    add(aten.embedding.default, lambda d: (_to(d, normal((50, 64), bf16, seed=1), randint((2, 3, 4), 50, 3, i32)), {}), exact=True, tag="3d_i32")
    add(aten.embedding.default, lambda d: (_to(d, normal((50, 64), bf16, seed=1), randint((9,), 50, 3), 0, False, False), {}), exact=True, tag="padding_idx_args")
    add(aten.embedding.default, lambda d: (_to(d, normal((1000, 4096), bf16, 0, 0.02, seed=1), randint((257,), 1000, 3)), {}), exact=True, tag="rows8k")
    add(aten.gather.default, lambda d: (_to(d, normal((5, 6, 7), f32, seed=1), 2, randint((5, 6, 3), 7, 3)), {}), exact=True, tag="3d_last")
    add(aten.gather.default, lambda d: (_to(d, normal((5, 6, 7), f32, seed=1), 1, randint((4, 9, 7), 6, 3)), {}), exact=True, tag="3d_mid_smaller")
    add(aten.gather.default, lambda d: ([normal((64, 20), f32, seed=1).to(d).t(), 1, randint((64, 20), 64, 3).to(d).t()], {}), exact=True, tag="transposed")
    add(aten.gather.default, lambda d: (_to(d, normal((20, 64), f32, seed=1), 1, torch.empty(20, 0, dtype=i64)), {}), exact=True, tag="empty_index")
    add(aten.gather.default, lambda d: (_to(d, torch.tensor(4.0), 0, torch.tensor(0)), {}), exact=True, tag="0d")
    add(aten.gather.default, lambda d: (_to(d, normal((256, 512), f32, seed=1), 1, randint((256, 512), 512, 3)), {"sparse_grad": False}), exact=True, tag="vec_path")
    return C


class CaseTest(Test):
    """Test over a Case: arguments are (re)drawn lazily from the seeded generator, so a
    suite of multi-gigabyte cases holds no tensors until a test is read."""

    def __init__(self, case, device):
        super().__init__()
        self.case = case
        self.device = device
        self._pending_kwargs = None

    @property
    def args(self):
        args, self._pending_kwargs = self.case.make(self.device)
        return list(args)

    @property
    def kwargs(self):
        kw, self._pending_kwargs = self._pending_kwargs, None
        return dict(kw) if kw is not None else dict(self.case.make(self.device)[1])


def sibling_perf_cases(scale: float = 1.0) -> List[Case]:
    """One timed case for each functional overload that has no headline row of its own, so that
    the evaluator's geometric mean over operators is defined for the whole suite.  They are not
    part of the headline measurement."""
    rows = max(8, int(4096 * scale))
    f16, bf16 = torch.float16, torch.bfloat16
    x = lambda seed, dt=f16: normal((rows, 4096), dt, seed=seed)
    row = lambda seed, dt=f16: normal((4096,), dt, seed=seed)
    return [
        Case("V.minimum", aten.minimum.default, lambda d: (_to(d, x(1), x(2)), {})),
        Case("V.clamp_min", aten.clamp_min.default, lambda d: (_to(d, x(1), -0.5), {})),
        Case("V.clamp_max", aten.clamp_max.default, lambda d: (_to(d, x(1), 0.5), {})),
        Case("V.clamp_tensor", aten.clamp.Tensor, lambda d: (_to(d, x(1), row(2) - 1, row(3) + 1), {})),
        Case("V.clamp_min_tensor", aten.clamp_min.Tensor, lambda d: (_to(d, x(1), row(2)), {})),
        Case("V.clamp_max_tensor", aten.clamp_max.Tensor, lambda d: (_to(d, x(1), row(2)), {})),
        Case("V.add_scalar", aten.add.Scalar, lambda d: (_to(d, x(1, bf16), 1.5), {})),
        Case("V.mul_scalar", aten.mul.Scalar, lambda d: (_to(d, x(1, bf16), 0.125), {})),
        Case("V.log_softmax", aten._log_softmax.default, lambda d: (_to(d, x(1, bf16), -1, False), {})),
        Case("V.mean_dim", aten.mean.dim, lambda d: (_to(d, x(1, bf16), [-1]), {})),
        Case("V.sum_all", aten.sum.default, lambda d: (_to(d, x(1, bf16)), {})),
        Case("V.mean_all", aten.mean.default, lambda d: (_to(d, x(1, bf16)), {})),
    ]


# functional overload -> its out= overload (BackendBench/scripts/op_map.py lists both on one `canonical:` line)
OUT_OVERLOADS = {
    aten.add.Tensor: aten.add.out, aten.mul.Tensor: aten.mul.out, aten.maximum.default: aten.maximum.out,
    aten.minimum.default: aten.minimum.out, aten.relu.default: aten.relu.out, aten.clamp.default: aten.clamp.out,
    aten.clamp.Tensor: aten.clamp.Tensor_out, aten.clamp_min.default: aten.clamp_min.out, aten.clamp_max.default: aten.clamp_max.out,
    aten.where.self: aten.where.self_out, aten.add.Scalar: aten.add.Scalar_out, aten.mul.Scalar: aten.mul.Scalar_out,
    aten.sum.dim_IntList: aten.sum.IntList_out, aten.sum.default: aten.sum.out, aten.mean.dim: aten.mean.out,
    aten.mean.default: aten.mean.dtype_out, aten.amax.default: aten.amax.out, aten.argmax.default: aten.argmax.out,
    aten._softmax.default: aten._softmax.out, aten._log_softmax.default: aten._log_softmax.out,
    aten.native_layer_norm.default: aten.native_layer_norm.out, aten.mm.default: aten.mm.out, aten.addmm.default: aten.addmm.out,
    aten.index_select.default: aten.index_select.out, aten.embedding.default: aten.embedding.out, aten.gather.default: aten.gather.out,
}


def out_perf_cases(scale: float = 1.0) -> List[Case]:
    """One timed case per out= overload: the headline row (or the sibling row) of its functional overload with
    an `out` of the result's shape, dtype and layout added - the case in which the kernels write into `out`
    directly, so the row should cost what the functional one does.  The result's shape comes from running the
    functional overload on meta tensors: nothing is computed to build the case."""
    seen, cases = set(), []
    for case in perf_cases(scale) + sibling_perf_cases(scale):
        out_op = OUT_OVERLOADS.get(case.op)
        if out_op is None or out_op in seen:
            continue
        seen.add(out_op)

        def make(device, case=case):
            args, kwargs = case.make(device)
            meta = lambda v: v.to("meta") if isinstance(v, torch.Tensor) else v
            res = case.op(*[meta(a) for a in args], **{k: meta(v) for k, v in kwargs.items()})
            dev = next(a.device for a in args if isinstance(a, torch.Tensor))
            fresh = lambda r: torch.empty_strided(r.shape, r.stride(), dtype=r.dtype, device=dev)
            if isinstance(res, (tuple, list)):
                return args, {**kwargs, **{f"out{i}": fresh(r) for i, r in enumerate(res)}}
            return args, {**kwargs, "out": fresh(res)}

        cases.append(Case("O." + case.key.split(".", 1)[1] + "_out", out_op, make, work=case.work, bound=case.bound,
                          exact=case.exact, note=f"out= form of {case.key}"))
    return cases


def _as_test(case, device):
    return CaseTest(case, device)


def BaselineTestSuite(device="cuda", scale=1.0, filter=None):
    """OpTests over the slots: edge cases as correctness tests, headline rows as
    performance tests.  `filter`: list of operator names matched exactly, with or without
    the overload ("_softmax", "add.Tensor"), as the reference's OpInfo suite matches --ops
    (BackendBench/suite/opinfo.py:91)."""
    per_op = {}
    for case in edge_cases():
        if device != "cpu" and case.extra.get("cpu_reference_only"):
            continue
        per_op.setdefault(case.op, ([], []))[0].append(case)
    for case in perf_cases(scale):
        per_op.setdefault(case.op, ([], []))[1].append(case)
    for case in sibling_perf_cases(scale):
        if not per_op.setdefault(case.op, ([], []))[1]:
            per_op[case.op][1].append(case)
    if device != "cpu":   # on the GPU only (the CPU suite is the oracle's; it pins functional overloads)
        for case in out_perf_cases(scale):
            per_op.setdefault(case.op, ([], []))[1].append(case)
        for case in out_perf_cases(min(scale, 0.02)):   # the same call at a small size as the correctness test
            per_op[case.op][0].append(case)
    optests = []
    for op, (edges, perfs) in per_op.items():
        name = op.__name__
        if filter and name not in filter and name.split(".")[0] not in filter:
            continue
        optests.append(OpTest(get_operator(op), [_as_test(c, device) for c in edges],
                              [_as_test(c, device) for c in perfs]))
    return TestSuite(f"baseline_{device}", optests)
