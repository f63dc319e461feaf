"""add.Tensor / mul.Tensor / maximum / relu / clamp / where.self on the HIP elementwise kernels.

Each function takes exactly the arguments of the ATen overload whose slot it fills
(reference: BackendBench/backends/directory.py:96-100 loads `<folder>_kernel_impl`,
BackendBench/eval.py:99-102 calls it as `impl(*args, **kwargs)`).
"""

import math

import torch

from .. import _lib
from ._common import (cast, copy_into, dense, device_managed, launch, new_dense, new_result, offer_out, result_like,
                      withdraw_out)


def _out_like_inputs(shape, dtype, inputs):
    """Output buffer: keeps a permuted-dense layout shared by the full-shape inputs (what
    ATen's TensorIterator does), row-major otherwise."""
    lead = None
    for t in inputs:
        if t.shape == shape:
            if lead is None:
                lead = t
            elif t.stride() != lead.stride():
                lead = None
                break
    if lead is not None:
        out = result_like(lead, dtype)
        if lead.is_contiguous() or out.stride() == lead.stride():  # preserve_format: dense permutations survive
            return out
    return new_result(shape, dtype, inputs[0].device)


def _is_permuted_dense(t):
    """True when `t` is a permutation of a dense tensor (no gaps, no overlap)."""
    expect = 1
    for size, stride in sorted(zip(t.shape, t.stride()), key=lambda p: p[1]):
        if size == 1:
            continue
        if stride != expect:
            return False
        expect *= size
    return True


def _align_layouts(shape, tensors):
    """Full-shape operands that disagree on layout run on the strided kernel, where the odd one is
    read one scattered element per lane.  When some operand is row-major and another is a permuted
    dense tensor whose last dim is not its contiguous one (a batched transpose, a channels-last
    view), the permuted one is made row-major first with the tiled transposing copy: two coalesced
    passes instead of one scattered pass.  Small problems keep the single pass: when the whole
    operand is a couple of MB the second launch costs more than the scatter, and transposed
    matrices of up to 128 KB each (attention heads) stay in cache while their lines are picked apart."""
    full = [t for t in tensors if t.shape == shape]
    if len(full) < 2 or len(shape) < 2 or shape[-1] == 1 or not any(t.is_contiguous() for t in full):
        return tensors
    esize = max(t.element_size() for t in full)
    if shape.numel() * esize <= (2 << 20):
        return tensors
    small_matrices = shape[-1] * shape[-2] * esize <= (128 << 10)
    out = []
    for t in tensors:
        if t.shape == shape and t.stride(-1) != 1 and not t.is_contiguous() and _is_permuted_dense(t):
            if not (small_matrices and t.transpose(-1, -2).is_contiguous()):
                t = dense(t)
        out.append(t)
    return out


def _broadcast_shape(*shapes):
    """torch.broadcast_shapes without its Python-side overhead (it costs more than a kernel launch)."""
    n = 0
    for s in shapes:
        if len(s) > n:
            n = len(s)
    out = [1] * n
    for s in shapes:
        off = n - len(s)
        for i, v in enumerate(s):
            cur = out[off + i]
            if cur == v or v == 1:
                continue
            if cur == 1:
                out[off + i] = v
            else:
                raise RuntimeError(f"The size of tensor a ({cur}) must match the size of tensor b ({v}) at "
                                   f"non-singleton dimension {off + i}")
    return torch.Size(out)


def _desc_as(t, shape):
    """Descriptor of `t` broadcast to `shape` (stride 0 on the broadcast dims), without expand()."""
    if t.shape == shape:
        return _lib.desc(t)
    off = len(shape) - t.dim()
    strides = [0] * off + [0 if n == 1 and shape[off + i] != 1 else st
                           for i, (n, st) in enumerate(zip(t.shape, t.stride()))]
    return _lib.desc(t, shape, strides)


def _alpha_args(dtype, alpha):
    if dtype.is_floating_point:
        return float(alpha), 0
    if isinstance(alpha, float) and not float(alpha).is_integer():
        raise RuntimeError("For integral input tensors, argument alpha must not be a floating point number.")
    return 0.0, int(alpha)


def _as_operand(self, other):
    """A Python number as second operand (the dispatcher unwraps the 0-d tensor that
    add.Scalar / `x *= 2` build) becomes a 0-d tensor of the promoted dtype on self's device."""
    if isinstance(other, torch.Tensor):
        return other
    return torch.full((), other, dtype=torch.result_type(self, other), device=self.device)


_MIXED_OPS = (_lib.ADD, _lib.MUL)
_HALF = (torch.float16, torch.bfloat16)


def _one_fp32_one_half(da, db):
    return (da == torch.float32 and db in _HALF) or (db == torch.float32 and da in _HALF)


def _binary(op, a, b, alpha=1):
    b = _as_operand(a, b)
    dtype = a.dtype if a.dtype == b.dtype else torch.result_type(a, b)
    if dtype.is_complex:
        raise NotImplementedError(f"mi355 backend: binary ops on {dtype} are not supported")
    if dtype == torch.bool:  # or / and / or: compute in u8, any non-zero is True
        return cast(_binary(op, cast(a, torch.uint8), cast(b, torch.uint8), 1 if alpha else 0), torch.bool)
    shape = a.shape if a.shape == b.shape else _broadcast_shape(a.shape, b.shape)
    if not (dtype == torch.float32 and op in _MIXED_OPS and _one_fp32_one_half(a.dtype, b.dtype)):
        a = cast(a, dtype)   # fp32 (+|*) f16 / bf16 is widened inside the kernel, everything else here
        b = cast(b, dtype)
    if a.stride() != b.stride():
        a, b = _align_layouts(shape, (a, b))
    out = _out_like_inputs(shape, dtype, (a, b))
    if out.numel() == 0:
        return out
    alpha_f, alpha_i = _alpha_args(dtype, alpha)
    launch("mi355_binary", op, _desc_as(a, shape), _desc_as(b, shape), alpha_f, alpha_i, _lib.desc(out))
    return out


def _dense_no_overlap(t):
    """Every element at its own address and no gaps: strides sorted ascending equal the running product of sizes."""
    expect = 1
    for size, stride in sorted(((sz, st) for sz, st in zip(t.shape, t.stride()) if sz != 1), key=lambda p: p[1]):
        if stride != expect:
            return False
        expect *= size
    return True


def _check_inplace_overlap(self, other=None):
    """ATen's refusals for a written-to tensor (TensorIterator's memory-overlap checks): `self` expanded
    over a stride-0 dim has several elements at one address; `other` sharing part of self's memory under
    another layout (x.add_(x.t()), x.add_(x[0])) would be read after it was overwritten."""
    if self.numel() == 0:
        return
    if any(sz > 1 and st == 0 for sz, st in zip(self.shape, self.stride())):
        raise RuntimeError("unsupported operation: more than one element of the written-to tensor refers to a single "
                           "memory location. Please clone() the tensor before performing the operation.")
    if not isinstance(other, torch.Tensor) or other.numel() == 0 or other.device != self.device:
        return
    if other.untyped_storage().data_ptr() != self.untyped_storage().data_ptr():
        return
    if not (_dense_no_overlap(self) and _dense_no_overlap(other)):
        return  # ATen calls these "too hard" and lets them through
    a0, b0 = self.data_ptr(), other.data_ptr()
    a1, b1 = a0 + self.numel() * self.element_size(), b0 + other.numel() * other.element_size()
    same_range = a0 == b0 and a1 == b1
    if (same_range and self.stride() != other.stride()) or (not same_range and a0 < b1 and b0 < a1):
        raise RuntimeError("unsupported operation: some elements of the input tensor and the written-to tensor refer to "
                           "a single memory location. Please clone() the tensor before performing the operation.")


def _binary_inplace(op, functional, self, other, **kw):
    """self (op)= other: the result type must be castable to self's dtype and broadcasting must
    not change self's shape, as for every ATen in-place overload.  `functional` is the
    out-of-place wrapper, used when the arithmetic dtype differs from self's or self is on the CPU."""
    _check_inplace_overlap(self, other)
    other = _as_operand(self, other)
    dtype = self.dtype if self.dtype == other.dtype else torch.result_type(self, other)
    full = self.shape if self.shape == other.shape else _broadcast_shape(self.shape, other.shape)
    if full != self.shape:
        raise RuntimeError(f"output with shape {list(self.shape)} doesn't match the broadcast shape {list(full)}")
    if dtype != self.dtype and not torch.can_cast(dtype, self.dtype):
        raise RuntimeError(f"result type {str(dtype).replace('torch.', '').capitalize()} can't be cast to the "
                           f"desired output type {str(self.dtype).replace('torch.', '').capitalize()}")
    if dtype != self.dtype or dtype == torch.bool or not self.is_cuda:
        return copy_into_any(self, functional(self, other, **kw))
    if self.numel() == 0:
        return self
    alpha_f, alpha_i = _alpha_args(dtype, kw.get("alpha", 1))
    b = other if other.is_cuda else other.to(self.device)
    if not (op in _MIXED_OPS and _one_fp32_one_half(dtype, b.dtype)):
        b = cast(b, dtype)
    mine = _lib.desc(self)
    launch("mi355_binary", op, mine, _desc_as(b, self.shape), alpha_f, alpha_i, mine)
    return self


def _is_gpu_tensor(t):
    return t.device.type == "cuda"


def copy_into_any(dst, src):
    """dst[...] = src across devices: our copy kernel on the GPU, torch's transfer otherwise."""
    if dst.is_cuda and src.is_cuda:
        if dst.numel():
            launch("mi355_copy", _desc_as(src, dst.shape), _lib.desc(dst))
    else:
        dst.copy_(src)  # host <-> device transfer (only reached with CPU tensors)
    return dst


@device_managed
def add(self, other, *, alpha=1):
    """aten.add.Tensor: self + alpha * other."""
    return _binary(_lib.ADD, self, other, alpha)


def add_(self, other, *, alpha=1):
    """aten.add_.Tensor"""
    return _binary_inplace(_lib.ADD, add, self, other, alpha=alpha)


@device_managed
def mul(self, other):
    """aten.mul.Tensor"""
    return _binary(_lib.MUL, self, other)


def mul_(self, other):
    """aten.mul_.Tensor"""
    return _binary_inplace(_lib.MUL, mul, self, other)


@device_managed
def maximum(self, other):
    """aten.maximum.default: NaN in either operand wins."""
    return _binary(_lib.MAXIMUM, self, other)


@device_managed
def minimum(self, other):
    """aten.minimum.default: NaN in either operand wins."""
    return _binary(_lib.MINIMUM, self, other)


_C_NAMES = {torch.uint8: "uint8_t", torch.int8: "int8_t", torch.int16: "int16_t", torch.int32: "int", torch.int64: "int64_t"}


def _unary(op, x, out_dtype, bounds=0, lo=None, hi=None, inplace=False):
    x = cast(x, out_dtype)
    out = x if inplace else result_like(x, out_dtype)  # preserve_format: dense permutations keep their layout
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
        # ATen refuses a bound the tensor's dtype cannot hold (c10::overflows: a negative bound on an
        # unsigned dtype wraps, down to -max); past that the kernel's narrowing would wrap it silently.
        info = torch.iinfo(out_dtype)
        floor = -info.max if info.min == 0 else info.min
        for bound in (lo_i, hi_i):
            if not floor <= bound <= info.max:
                raise RuntimeError(f"value cannot be converted to type {_C_NAMES.get(out_dtype, str(out_dtype))} without overflow")
    launch("mi355_unary", op, _lib.desc(x), bounds, lo_f, hi_f, lo_i, hi_i, _lib.desc(out))
    return out


def _check_relu_dtype(t):
    if t.dtype == torch.bool or t.dtype.is_complex:
        raise RuntimeError(f"relu is not implemented for {t.dtype}")


@device_managed
def relu(self):
    """aten.relu.default"""
    _check_relu_dtype(self)
    return _unary(_lib.RELU, self, self.dtype)


def relu_(self):
    """aten.relu_.default"""
    _check_relu_dtype(self)
    _check_inplace_overlap(self)
    if not _is_gpu_tensor(self):
        return copy_into_any(self, relu(self))
    _unary(_lib.RELU, self, self.dtype, inplace=True)
    return self


def _clamp_dtype(self, bounds):
    """Result dtype of clamp with Python-number bounds: a float bound lifts an integer tensor to
    the default float dtype, anything else keeps self's dtype (result_type of a dimensioned
    tensor with scalars)."""
    dtype = self.dtype
    if not dtype.is_floating_point:
        for bound in bounds:
            if isinstance(bound, float):
                dtype = torch.get_default_dtype()
            elif bound is not None and not isinstance(bound, (int, bool)):
                dtype = torch.result_type(torch.empty((), dtype=dtype, device="meta").expand(1), bound)
    if dtype == torch.bool or dtype.is_complex:
        raise NotImplementedError(f"mi355 backend: clamp on {dtype} is not supported")
    return dtype


@device_managed
def clamp(self, min=None, max=None):
    """aten.clamp.default: Scalar bounds; at least one must be given."""
    if min is None and max is None:
        raise RuntimeError("torch.clamp: At least one of 'min' or 'max' must not be None")
    bounds = (1 if min is not None else 0) | (2 if max is not None else 0)
    return _unary(_lib.CLAMP, self, _clamp_dtype(self, (min, max)), bounds, min, max)


def clamp_(self, min=None, max=None):
    """aten.clamp_.default"""
    if min is None and max is None:
        raise RuntimeError("torch.clamp: At least one of 'min' or 'max' must not be None")
    _check_inplace_overlap(self)
    dtype = _clamp_dtype(self, (min, max))
    if not torch.can_cast(dtype, self.dtype):
        raise RuntimeError(f"result type {str(dtype).replace('torch.', '').capitalize()} can't be cast to the "
                           f"desired output type {str(self.dtype).replace('torch.', '').capitalize()}")
    if dtype != self.dtype or not _is_gpu_tensor(self):
        return copy_into_any(self, clamp(self, min, max))
    bounds = (1 if min is not None else 0) | (2 if max is not None else 0)
    _unary(_lib.CLAMP, self, dtype, bounds, min, max, inplace=True)
    return self


@device_managed
def clamp_min(self, min):
    """aten.clamp_min.default"""
    return _unary(_lib.CLAMP, self, _clamp_dtype(self, (min,)), 1, min, None)


@device_managed
def clamp_max(self, max):
    """aten.clamp_max.default"""
    return _unary(_lib.CLAMP, self, _clamp_dtype(self, (max,)), 2, None, max)


@device_managed
def clamp_tensor(self, min=None, max=None):
    """aten.clamp.Tensor: tensor bounds, min(max(self, lo), hi) with NaN propagation."""
    if min is None and max is None:
        raise RuntimeError("torch.clamp: At least one of 'min' or 'max' must not be None")
    if min is not None and max is not None and self.dtype == min.dtype == max.dtype and self.is_cuda \
            and not self.dtype.is_complex and self.dtype != torch.bool:
        # both bounds, no promotion: one fused pass
        if self.shape == min.shape == max.shape:
            shape = self.shape
        else:
            shape = _broadcast_shape(self.shape, min.shape, max.shape)
        x, lo, hi = self, min, max
        if not (x.stride() == lo.stride() == hi.stride()):
            x, lo, hi = _align_layouts(shape, (x, lo, hi))
        out = _out_like_inputs(shape, self.dtype, (x, lo, hi))
        if out.numel():
            launch("mi355_clamp_tensor", _desc_as(x, shape), _desc_as(lo, shape), _desc_as(hi, shape), _lib.desc(out))
        return out
    out = self
    if min is not None:
        out = _binary(_lib.MAXIMUM, out, min)
    if max is not None:
        out = _binary(_lib.MINIMUM, out, max)
    return out


@device_managed
def where(condition, self, other):
    """aten.where.self: bit-exact select with broadcasting."""
    if condition.dtype not in (torch.bool, torch.uint8):
        raise RuntimeError(f"where expected condition to be a boolean tensor, but got a tensor with dtype {condition.dtype}")
    dtype = self.dtype if self.dtype == other.dtype else torch.result_type(self, other)
    if condition.shape == self.shape == other.shape:
        shape = self.shape
    else:
        shape = _broadcast_shape(condition.shape, self.shape, other.shape)
    a = cast(self, dtype)
    b = cast(other, dtype)
    if not (condition.stride() == a.stride() == b.stride()):
        condition, a, b = _align_layouts(shape, (condition, a, b))
    out = _out_like_inputs(shape, dtype, (condition, a, b))
    if out.numel() == 0:
        return out
    launch("mi355_where", _desc_as(condition, shape), _desc_as(a, shape), _desc_as(b, shape), _lib.desc(out))
    return out


def _inplace_from(functional, name):
    """`self = functional(self, ...)` for the in-place overloads with no kernel form of their own:
    the result must be castable to self's dtype and have self's shape, as ATen requires."""

    def impl(self, *args, **kwargs):
        res = functional(self, *args, **kwargs)
        if res.shape != self.shape:
            raise RuntimeError(f"output with shape {list(self.shape)} doesn't match the broadcast shape {list(res.shape)}")
        if not torch.can_cast(res.dtype, self.dtype):
            raise RuntimeError(f"result type {str(res.dtype).replace('torch.', '').capitalize()} can't be cast to the "
                               f"desired output type {str(self.dtype).replace('torch.', '').capitalize()}")
        return copy_into_any(self, res if res.device == self.device else res.to(self.device))

    impl.__name__ = name
    impl.__doc__ = f"in-place variant of {functional.__name__}"
    return impl


def clamp_min_(self, min):
    """aten.clamp_min_.default"""
    return clamp_(self, min, None)


def clamp_max_(self, max):
    """aten.clamp_max_.default"""
    return clamp_(self, None, max)


def clamp_min_tensor(self, min):
    """aten.clamp_min.Tensor: max(self, min) with NaN propagation and maximum's type promotion."""
    return maximum(self, min)


def clamp_max_tensor(self, max):
    """aten.clamp_max.Tensor: min(self, max) with NaN propagation and minimum's type promotion."""
    return minimum(self, max)


def _shares_memory(out, args, kwargs):
    """True when `out` lives in the storage of some tensor argument (conservative: same storage = overlap)."""
    base = out.untyped_storage().data_ptr()
    for a in list(args) + list(kwargs.values()):
        if isinstance(a, torch.Tensor) and a.device == out.device and a.numel() and a.untyped_storage().data_ptr() == base:
            return True
    return False


def _call_into(functional, outs, args, kwargs):
    """functional(*args, **kwargs) with `outs` offered as result buffers (see _common.offer_out): GPU tensors
    that share no storage with an argument - a kernel writing its result over an operand it is still
    reading would be a race the functional form does not have."""
    direct = [o for o in outs if o.is_cuda and not _shares_memory(o, args, kwargs)]
    if len(direct) != len(outs):
        return functional(*args, **kwargs)
    offer_out(*direct)
    try:
        return functional(*args, **kwargs)
    finally:
        withdraw_out()


def _store_result(out, res):
    """`res` into `out` as ATen's out= overloads do: castable dtype, `out` resized when its shape differs."""
    if res is out:
        return out  # the kernel wrote into `out` itself
    if not torch.can_cast(res.dtype, out.dtype):
        raise RuntimeError(f"result type {str(res.dtype).replace('torch.', '').capitalize()} can't be cast to "
                           f"the desired output type {str(out.dtype).replace('torch.', '').capitalize()}")
    if tuple(out.shape) != tuple(res.shape):
        out.resize_(res.shape)
    if res.device != out.device:
        res = res.to(out.device)
    return copy_into_any(out, res)


def tuple_out_variant(functional, n):
    """`<op>.out(..., out0=, out1=, ...)` of an operator with `n` results (native_layer_norm.out): each result
    lands in its own out tensor - written there by the kernel when that tensor already has the result's shape,
    dtype and a dense layout, resized / cast by a copy otherwise; returns the out tensors."""

    def impl(*args, **kwargs):
        outs = [kwargs.pop(f"out{i}") for i in range(n)]
        results = _call_into(functional, outs, args, kwargs)
        for res, out in zip(results, outs):
            if res is not out and not torch.can_cast(res.dtype, out.dtype):
                raise RuntimeError(f"result type {str(res.dtype).replace('torch.', '').capitalize()} can't be cast to "
                                   f"the desired output type {str(out.dtype).replace('torch.', '').capitalize()}")
        return tuple(_store_result(out, res) for res, out in zip(results, outs))

    impl.__name__ = functional.__name__ + "_out"
    impl.__doc__ = f"out= variant of {functional.__name__} ({n} results)"
    return impl


def out_variant(functional):
    """`<op>.out(..., out=Tensor)` from the functional wrapper.  When `out` already has the result's shape and
    dtype, a dense layout and no memory in common with an argument, the kernel writes into it directly (the
    common case: same traffic as the functional form).  Otherwise the result is computed into a temporary,
    `out` is resized if its shape differs (as ATen does) and the copy kernel stores it with a cast."""

    def impl(*args, out, **kwargs):
        return _store_result(out, _call_into(functional, [out], args, kwargs))

    impl.__name__ = functional.__name__ + "_out"
    impl.__doc__ = f"out= variant of {functional.__name__}"
    return impl
