"""A second, tighter bar beside the reference's `atol = rtol = 1e-2` (BackendBench/eval.py:68-90).

The reference's tolerance cannot tell fp32 accumulation from bf16, nor fp64 from fp32.  `tight_check`
compares a result with the numpy float64 restatement of the operator (oracle/numpy_ref.py, on the inputs
exactly widened) at what the advertised arithmetic must reach:

    fp32 results:        |got - exact| <= 1e-5  * sqrt(L) * R
    fp64 results:        |got - exact| <= 1e-12 * sqrt(L) * R
    bf16 / f16 results:  the fp32 bound + 2 ulp of the output dtype at |exact|

L = the length of the reduction behind an output element (1 for elementwise), R = the natural scale of
its rounding error: |exact| where nothing cancels (elementwise, softmax), the root of the sum of the squared
terms where terms of both signs are added (sum, mean, mm, addmm), and for layer norm the size of the
products before the mean is taken out.  A bf16 (or, for f64, an fp32) accumulator misses these bounds by two
orders of magnitude; tests/test_oracle.py checks that on the CPU with a deliberately narrowed accumulator.
Test infrastructure only.
"""

import numpy as np
import torch

from oracle import numpy_ref


def np_of(t):
    if isinstance(t, torch.Tensor):
        if t.dtype in (torch.bfloat16, torch.float16, torch.float32):
            return t.double().numpy()
        return t.numpy()
    return t


def numpy_result(case, args, kwargs):
    n = case.op.__name__
    a = [np_of(x) for x in args]
    if n in ("add.Tensor", "add.Scalar"):
        return numpy_ref.add(a[0], a[1], kwargs.get("alpha", 1))
    if n in ("mul.Tensor", "mul.Scalar"):
        return numpy_ref.mul(a[0], a[1])
    if n in ("maximum.default", "clamp_min.Tensor"):
        return numpy_ref.maximum(*np.broadcast_arrays(a[0], a[1]))
    if n in ("minimum.default", "clamp_max.Tensor"):
        return numpy_ref.minimum(*np.broadcast_arrays(a[0], a[1]))
    if n == "clamp_min.default":
        return numpy_ref.clamp(a[0], a[1], None)
    if n == "clamp_max.default":
        return numpy_ref.clamp(a[0], None, a[1])
    if n == "clamp.Tensor":
        return numpy_ref.clamp_tensor(a[0], a[1], a[2] if len(a) > 2 else None)
    if n == "_log_softmax.default":
        return numpy_ref.log_softmax(a[0], a[1])
    if n == "relu.default":
        return numpy_ref.relu(a[0])
    if n == "clamp.default":
        return numpy_ref.clamp(a[0], *(a[1:] + [None, None])[:2])
    if n == "where.self":
        return numpy_ref.where(a[0], a[1], a[2])
    if n in ("sum.dim_IntList", "mean.dim", "amax.default"):
        fn = {"sum.dim_IntList": numpy_ref.sum_, "mean.dim": numpy_ref.mean, "amax.default": numpy_ref.amax}[n]
        dim = a[1] if len(a) > 1 else ([] if n == "amax.default" else None)
        return fn(a[0], dim, a[2] if len(a) > 2 else False)
    if n in ("sum.default", "mean.default"):
        return (numpy_ref.sum_ if n == "sum.default" else numpy_ref.mean)(a[0], None)
    if n == "argmax.default":
        return numpy_ref.argmax(a[0], a[1] if len(a) > 1 else None, a[2] if len(a) > 2 else False)
    if n == "_softmax.default":
        return numpy_ref.softmax(a[0], a[1]) if a[0].ndim else np.ones(())
    if n == "native_layer_norm.default":
        return numpy_ref.layer_norm(a[0], a[1], a[2], a[3], a[4])
    if n == "mm.default":
        return numpy_ref.mm(a[0], a[1])
    if n == "addmm.default":
        return numpy_ref.addmm(a[0], a[1], a[2], kwargs.get("beta", 1), kwargs.get("alpha", 1))
    if n == "index_select.default":
        return numpy_ref.index_select(a[0], a[1], a[2])
    if n == "embedding.default":
        return numpy_ref.embedding(a[0], a[1])
    if n == "gather.default":
        if a[0].ndim == 0:
            return a[0]
        return numpy_ref.gather(a[0], a[1], a[2])
    raise AssertionError(n)




_ULP_BITS = {torch.bfloat16: 8, torch.float16: 11}


def _ulp(ref, dtype):
    """Spacing of `dtype` at |ref| (normal range; the smallest normal's spacing below it)."""
    bits = _ULP_BITS[dtype]
    tiny = float(torch.finfo(dtype).tiny)
    mag = np.maximum(np.abs(ref), tiny)
    return np.exp2(np.floor(np.log2(mag)) - (bits - 1))


def _scale(name, a, kwargs, ref, which):
    """(L, R) for output number `which` of operator `name` (see the module docstring)."""
    sq = lambda v: np.square(np.abs(np.asarray(v, dtype=np.float64)))
    if name in ("add.Tensor", "add.Scalar"):
        return 2, np.abs(a[0]) + np.abs(kwargs.get("alpha", 1) * np.asarray(a[1], dtype=np.float64))
    if name in ("sum.dim_IntList", "mean.dim", "sum.default", "mean.default"):
        default = name.endswith(".default")
        dim = None if default else (a[1] if len(a) > 1 else None)
        keep = False if default else (a[2] if len(a) > 2 else False)
        x = np.asarray(a[0], dtype=np.float64)
        count = max(1, x.size // max(1, np.asarray(ref).size))
        r = np.sqrt(numpy_ref.sum_(sq(x), dim, keep))
        return count, r / count if name.startswith("mean") else r
    if name in ("_softmax.default",):
        return (a[0].shape[a[1]] if a[0].ndim else 1), np.abs(ref)
    if name == "_log_softmax.default":
        return (a[0].shape[a[1]] if a[0].ndim else 1), np.abs(ref) + 1.0
    if name == "native_layer_norm.default":
        x = np.asarray(a[0], dtype=np.float64)
        k = len(a[1])
        n = int(np.prod(a[1])) if k else 1
        axes = tuple(range(x.ndim - k, x.ndim))
        mean = x.mean(axis=axes, keepdims=True) if n else np.zeros(x.shape[: x.ndim - k] + (1,) * k)
        rstd = 1.0 / np.sqrt(x.var(axis=axes, keepdims=True) + a[4]) if n else mean
        if which == 0:
            w = np.abs(np.asarray(a[2], dtype=np.float64)) if a[2] is not None else 1.0
            b = np.abs(np.asarray(a[3], dtype=np.float64)) if a[3] is not None else 0.0
            return n, np.abs(ref) + b + (np.abs(x) + np.abs(mean)) * rstd * w
        if which == 1:
            return n, np.sqrt(sq(x).sum(axis=axes, keepdims=True)) / max(n, 1)
        return n, np.abs(ref) * (1.0 + sq(mean) * sq(rstd))
    if name in ("mm.default", "mm.dtype"):
        return a[0].shape[1], np.sqrt(numpy_ref.mm(sq(a[0]), sq(a[1])))
    if name in ("addmm.default", "addmm.dtype"):
        al, be = kwargs.get("alpha", 1), kwargs.get("beta", 1)
        prod = numpy_ref.mm(sq(a[1]), sq(a[2])) * float(al) ** 2
        c = sq(np.broadcast_to(a[0], prod.shape)) * float(be) ** 2 if be != 0 else 0.0
        return a[1].shape[1] + 1, np.sqrt(prod + c)
    return 1, np.abs(ref)


def tight_check(case, args, kwargs, got):
    """None when `got` (tensor or tuple of tensors, on any device) meets the tighter bar for `case.op` on the
    CPU copies `args` / `kwargs`; else a message naming the worst element.  Integer / bool / copied results
    are left to the exact comparison of the usual bar."""
    name = case.op.__name__
    if name in ("argmax.default", "index_select.default", "embedding.default", "gather.default", "where.self",
                "amax.default", "relu.default", "clamp.default", "clamp.Tensor", "clamp_min.default", "clamp_max.default",
                "clamp_min.Tensor", "clamp_max.Tensor", "maximum.default", "minimum.default"):
        return None  # selections and copies: exact by construction, compared bit for bit or by value elsewhere
    tensors = [x for x in args if isinstance(x, torch.Tensor)]
    if any(t.numel() == 0 or t.dim() == 0 for t in tensors[:1]) or any(t.numel() == 0 for t in tensors):
        return None  # empty and 0-d operands: nothing is accumulated; the usual bar covers them
    if kwargs.get("dtype") is not None and name.split(".")[0] in ("sum", "mean"):
        # ATen's definition: sum(x, dtype=d) = sum(x.to(d)) - the terms are rounded to d first
        args = [args[0].to(kwargs["dtype"])] + list(args[1:])
    a = [np_of(x) for x in args]
    want = numpy_result(case, args, kwargs)
    wants = list(want) if isinstance(want, (tuple, list)) else [want]
    gots = list(got) if isinstance(got, (tuple, list)) else [got]
    for which, (w, g) in enumerate(zip(wants, gots)):
        if not (isinstance(g, torch.Tensor) and g.dtype.is_floating_point) or g.numel() == 0:
            continue
        w = np.asarray(w, dtype=np.float64)
        gv = g.detach().cpu().double().numpy().reshape(w.shape)
        L, R = _scale(name, a, kwargs, w, which)
        R = np.broadcast_to(np.asarray(R, dtype=np.float64), w.shape) if np.ndim(R) else np.full(w.shape, float(R))
        unit = 1e-12 if g.dtype == torch.float64 else 1e-5
        # inputs narrower than the output (a bf16 sum returned in fp32) do not loosen the bar: the terms are exact
        with np.errstate(invalid="ignore", over="ignore"):
            tol = unit * np.sqrt(max(L, 1)) * R
            if g.dtype in _ULP_BITS:
                tol = tol + 2.0 * _ulp(w, g.dtype)
            finite = np.isfinite(w) & np.isfinite(R)
            err = np.abs(gv - w)
            bad = finite & ~(err <= tol)
        if bad.any():
            i = np.unravel_index(np.argmax(np.where(bad, err / np.maximum(tol, 1e-300), 0.0)), w.shape)
            return (f"{name} output {which} ({g.dtype}): |got - exact| = {err[i]:.3e} > {tol[i]:.3e} at {tuple(int(v) for v in i)} "
                    f"(exact {w[i]:.6g}, got {gv[i]:.6g}, L = {L}, {int(bad.sum())} of {w.size} elements over)")
    return None
