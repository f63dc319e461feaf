"""ATen-on-CPU reference for one operator call (test infrastructure, see oracle/__init__.py).

Follows BackendBench/eval.py:99-100 (`ref = op(*args, **kwargs)`) with the arguments moved
to the CPU, plus the two places where ATen's CPU and GPU kernels differ in *signature*
rather than in mathematics and the device convention is the one the backend follows:

* `_softmax` / `_log_softmax(x, dim, half_to_float=True)`: the CPU kernel refuses it; the reference value is
  `_softmax(x.float(), dim, False)` (the same mathematics: fp32 softmax of the upcast input).
* `native_layer_norm` on f16/bf16 input: the CPU kernel returns mean/rstd rounded to the
  input dtype, GPU kernels return them in fp32.  y comes from the plain call; mean/rstd come
  from the call on the fp32 upcast of the same input (identical statistics before rounding).
"""

import time

import torch


def to_cpu(obj):
    if isinstance(obj, torch.Tensor):
        return obj.detach().cpu()
    if isinstance(obj, (list, tuple)):
        return type(obj)(to_cpu(o) for o in obj)
    if isinstance(obj, dict):
        return {k: to_cpu(v) for k, v in obj.items()}
    return obj


def reference(op, args, kwargs=None):
    """Result of `op` on CPU copies of (args, kwargs), adapted as described above."""
    args = to_cpu(list(args))
    kwargs = to_cpu(dict(kwargs or {}))
    name = op.__name__
    if name in ("_softmax.default", "_log_softmax.default") and len(args) >= 3 and args[2]:
        return op(args[0].float(), args[1], False)
    if name == "native_layer_norm.default" and args[0].dtype in (torch.float16, torch.bfloat16):
        x, shape, w, b, eps = args
        y, _, _ = op(x, shape, w, b, eps)
        up = lambda t: t.float() if t is not None else None
        _, mean, rstd = op(x.float(), shape, up(w), up(b), eps)
        return y, mean, rstd
    return op(*args, **kwargs)


def raises(op, args, kwargs=None):
    """The exception type ATen's CPU kernel raises for this call, or None."""
    try:
        reference(op, args, kwargs)
    except Exception as exc:  # noqa: BLE001 - the type is the result
        return type(exc)
    return None


def time_call(op, args, kwargs=None, warmup=10, runs=100):
    """Mean seconds per call with the reference's CPU recipe (BackendBench/eval.py:149-159:
    `warmup` untimed calls, then `runs` timed with perf_counter)."""
    args = to_cpu(list(args))
    kwargs = to_cpu(dict(kwargs or {}))
    for _ in range(warmup):
        op(*args, **kwargs)
    t0 = time.perf_counter()
    for _ in range(runs):
        op(*args, **kwargs)
    return (time.perf_counter() - t0) / runs
