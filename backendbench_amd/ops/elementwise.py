"""add.Tensor / mul.Tensor / maximum / relu / clamp / where.self on the HIP elementwise kernels.

Each function takes exactly the arguments of the ATen overload whose slot it fills
(reference: BackendBench/backends/directory.py:96-100 loads `<folder>_kernel_impl`,
BackendBench/eval.py:99-102 calls it as `impl(*args, **kwargs)`).
"""

import math

import torch

from .. import _lib
from ._common import cast, device_managed, launch


def _out_like_inputs(shape, dtype, inputs):
    """Output buffer: keeps a permuted-dense layout shared by the full-shape inputs (what
    ATen's TensorIterator does), row-major otherwise."""
    lead = None
    for t in inputs:
        if tuple(t.shape) == tuple(shape):
            if lead is None:
                lead = t
            elif t.stride() != lead.stride():
                lead = None
                break
    if lead is not None and not lead.is_contiguous():
        out = torch.empty_like(lead, dtype=dtype)  # preserve_format: dense permutations survive
        if out.stride() == lead.stride():
            return out
    return torch.empty(shape, dtype=dtype, device=inputs[0].device)


def _binary(op, a, b, alpha=1):
    dtype = torch.result_type(a, b)
    if dtype.is_complex:
        raise NotImplementedError(f"mi355 backend: binary ops on {dtype} are not supported")
    if dtype == torch.bool:  # or / and / or: compute in u8, any non-zero is True
        return cast(_binary(op, cast(a, torch.uint8), cast(b, torch.uint8), 1 if alpha else 0), torch.bool)
    shape = torch.broadcast_shapes(a.shape, b.shape)
    a = cast(a, dtype)
    b = cast(b, dtype)
    out = _out_like_inputs(shape, dtype, (a, b))
    if out.numel() == 0:
        return out
    if dtype.is_floating_point:
        alpha_f, alpha_i = float(alpha), 0
    else:
        if isinstance(alpha, float) and not float(alpha).is_integer():
            raise RuntimeError("For integral input tensors, argument alpha must not be a floating point number.")
        alpha_f, alpha_i = 0.0, int(alpha)
    launch("mi355_binary", op, _lib.desc(a.expand(shape)), _lib.desc(b.expand(shape)), alpha_f, alpha_i,
           _lib.desc(out))
    return out


@device_managed
def add(self, other, *, alpha=1):
    """aten.add.Tensor: self + alpha * other."""
    return _binary(_lib.ADD, self, other, alpha)


@device_managed
def mul(self, other):
    """aten.mul.Tensor"""
    return _binary(_lib.MUL, self, other)


@device_managed
def maximum(self, other):
    """aten.maximum.default: NaN in either operand wins."""
    return _binary(_lib.MAXIMUM, self, other)


def _unary(op, x, out_dtype, bounds=0, lo=None, hi=None):
    x = cast(x, out_dtype)
    out = _out_like_inputs(x.shape, out_dtype, (x,))
    if out.numel() == 0:
        return out
    if out_dtype.is_floating_point:
        lo_f = float(lo) if lo is not None else 0.0
        hi_f = float(hi) if hi is not None else 0.0
        lo_i = hi_i = 0
    else:
        lo_f = hi_f = 0.0
        lo_i = int(lo) if lo is not None else 0
        hi_i = int(hi) if hi is not None else 0
    launch("mi355_unary", op, _lib.desc(x), bounds, lo_f, hi_f, lo_i, hi_i, _lib.desc(out))
    return out


@device_managed
def relu(self):
    """aten.relu.default"""
    if self.dtype == torch.bool or self.dtype.is_complex:
        raise RuntimeError(f"relu is not implemented for {self.dtype}")
    return _unary(_lib.RELU, self, self.dtype)


@device_managed
def clamp(self, min=None, max=None):
    """aten.clamp.default: Scalar bounds; at least one must be given."""
    if min is None and max is None:
        raise RuntimeError("torch.clamp: At least one of 'min' or 'max' must not be None")
    dtype = self.dtype
    for bound in (min, max):
        if bound is not None:
            dtype = torch.result_type(torch.empty((), dtype=dtype, device="meta").expand(1), bound)
    if dtype == torch.bool or dtype.is_complex:
        raise NotImplementedError(f"mi355 backend: clamp on {dtype} is not supported")
    bounds = (1 if min is not None else 0) | (2 if max is not None else 0)
    return _unary(_lib.CLAMP, self, dtype, bounds, min, max)


@device_managed
def where(condition, self, other):
    """aten.where.self: bit-exact select with broadcasting."""
    if condition.dtype not in (torch.bool, torch.uint8):
        raise RuntimeError(f"where expected condition to be a boolean tensor, but got a tensor with dtype {condition.dtype}")
    dtype = torch.result_type(self, other)
    shape = torch.broadcast_shapes(condition.shape, self.shape, other.shape)
    a = cast(self, dtype)
    b = cast(other, dtype)
    out = _out_like_inputs(shape, dtype, (condition, a, b))
    if out.numel() == 0:
        return out
    launch("mi355_where", _lib.desc(condition.expand(shape)), _lib.desc(a.expand(shape)),
           _lib.desc(b.expand(shape)), _lib.desc(out))
    return out
