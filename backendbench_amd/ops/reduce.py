"""sum / mean / amax / argmax, _softmax and native_layer_norm on the HIP row kernels.

Every kernel sees a dense [outer, red, inner] view.  When the reduced dims are adjacent in
a contiguous tensor that view is free; otherwise the operand is permuted/densified once
with the copy kernel.
"""

import torch

from .. import _lib
from ._common import cast, copy_into, dense, device_managed, launch, new_dense, new_result, norm_dim, prod

_NATIVE_IN = (torch.float32, torch.float16, torch.bfloat16, torch.float64, torch.int32, torch.int64)
_SMALL_INT = (torch.int16, torch.int8, torch.uint8, torch.bool)


def _norm_dims(dim, ndim):
    if dim is None:
        return list(range(ndim))
    if isinstance(dim, int):
        dim = [dim]
    dims = sorted({norm_dim(d, ndim) for d in dim}) if ndim > 0 else []
    if len(dims) != len(list(dim)) and ndim > 0:
        raise RuntimeError("dim appears multiple times in the list of dims")
    if not dims:
        return list(range(ndim))
    return dims


def _memory_view3(x, dims):
    """(outer, red, inner) when `x` is a permuted dense tensor whose reduced dims are adjacent *in
    memory* and whose kept dims lie in memory in their logical order (e.g. the last dim of a
    transposed matrix): the reduction then runs on the memory as it is, no copy.  None otherwise."""
    live = [d for d in range(x.dim()) if x.shape[d] != 1]
    order = sorted(live, key=lambda d: -x.stride(d))          # outermost in memory first
    expect = 1
    for d in reversed(order):
        if x.stride(d) != expect:
            return None
        expect *= x.shape[d]
    red_pos = [i for i, d in enumerate(order) if d in dims]
    if not red_pos or red_pos != list(range(red_pos[0], red_pos[-1] + 1)):
        return None
    kept = [d for d in order if d not in dims]
    if kept != sorted(kept):
        return None
    outer = prod(x.shape[d] for d in order[: red_pos[0]])
    red = prod(x.shape[d] for d in order[red_pos[0] : red_pos[-1] + 1])
    inner = prod(x.shape[d] for d in order[red_pos[-1] + 1 :])
    return outer, red, inner


def _view3(x, dims):
    """(dense tensor, outer, red, inner) with the dims in `dims` reduced."""
    nd = x.dim()
    if nd == 0:
        return dense(x), 1, 1, 1
    if not x.is_contiguous():
        mem = _memory_view3(x, dims)
        if mem is not None:
            return (x,) + mem
    adjacent = dims == list(range(dims[0], dims[-1] + 1))
    if adjacent:
        xd = dense(x)
        shape = x.shape
        return xd, prod(shape[: dims[0]]), prod(shape[dims[0] : dims[-1] + 1]), prod(shape[dims[-1] + 1 :])
    kept = [d for d in range(nd) if d not in dims]
    xp = x.permute(kept + dims)
    xd = copy_into(new_dense(xp.shape, x.dtype, x.device), xp)
    return xd, prod(x.shape[d] for d in kept), prod(x.shape[d] for d in dims), 1


def _out_shape(x, dims, keepdim):
    if x.dim() == 0:
        return []
    if keepdim:
        return [1 if d in dims else s for d, s in enumerate(x.shape)]
    return [s for d, s in enumerate(x.shape) if d not in dims]


def _adjacent_runs(dims):
    runs = [[dims[0]]]
    for d in dims[1:]:
        if d == runs[-1][-1] + 1:
            runs[-1].append(d)
        else:
            runs.append([d])
    return runs


def _row_workspace(rows, n, x):
    """Scratch for the split form of softmax / layer norm over few, very long rows (None when the
    library does not split this shape).  The planning call is skipped for shapes it never splits."""
    if rows >= 64 or n < 32768:
        return None, 0
    nbytes = _lib.load().mi355_row_workspace_bytes(rows, n, _lib.dtype_code(x.dtype))
    if nbytes <= 0:
        return None, 0
    return torch.empty(nbytes, dtype=torch.uint8, device=x.device), nbytes


def _run_reduce(op, x, dims, keepdim, out_dtype):
    """x: tensor of a natively reducible dtype with numel > 0 and red > 0."""
    if len(dims) > 1 and op in (_lib.SUM, _lib.MEAN, _lib.AMAX):
        runs = _adjacent_runs(dims)
        if len(runs) > 1 and (x.is_contiguous() or _memory_view3(x, dims) is None):
            # Reduced dims that are not neighbours (a batch-norm style sum over N, H, W): the
            # innermost run first, then the rest on the much smaller intermediate (kept in fp32 /
            # int64 so that it is rounded once) - one pass over x instead of a permuting copy + a pass.
            if out_dtype.is_floating_point:
                inter = torch.float64 if x.dtype == torch.float64 else torch.float32
            else:
                inter = out_dtype
            first = _run_reduce(op, x, runs[-1], True, inter)
            rest = [d for run in runs[:-1] for d in run]
            res = _run_reduce(op, first, rest, True, inter)
            return cast(res, out_dtype).view(_out_shape(x, dims, keepdim))
    xd, outer, red, inner = _view3(x, dims)
    if inner > 1 and red >= 256 and xd.numel() >= 131072 and (inner < 64 or outer * ((inner + 63) // 64) < 64):
        # A long reduced axis over few columns: the column kernels run lanes along `inner`, so most
        # of a wave idles (inner < 64) or a handful of blocks walk the axis.  One transposing copy
        # turns the columns into rows for the row kernels ([1000000, 8] f16 summed over dim 0:
        # 732 us on the column kernel).  Indices along the reduced axis are unchanged by it.
        xd = dense(xd.as_strided((outer, red, inner), (red * inner, inner, 1)).transpose(1, 2))  # xd's memory is dense in this order
        outer, inner = outer * inner, 1
    out = new_result(_out_shape(x, dims, keepdim), out_dtype, x.device)
    lib = _lib.load()
    in_code, out_code = _lib.dtype_code(xd.dtype), _lib.dtype_code(out_dtype)
    ws_bytes = lib.mi355_reduce_workspace_bytes(op, in_code, outer, red, inner)
    ws = new_dense((ws_bytes,), torch.uint8, x.device) if ws_bytes else None
    launch("mi355_reduce", op, xd.data_ptr(), in_code, outer, red, inner, out.data_ptr(), out_code,
           ws.data_ptr() if ws is not None else None, ws_bytes)
    return out


def _sum_like(op, x, dim, keepdim, dtype, name):
    dims = _norm_dims(dim, x.dim())
    if dtype is None:
        if x.dtype.is_floating_point:
            dtype = x.dtype
        elif op == _lib.MEAN:
            raise RuntimeError(
                f"{name}(): could not infer output dtype. Input dtype must be either a floating point or "
                f"complex dtype. Got: {str(x.dtype).replace('torch.', '').capitalize()}")
        else:
            dtype = torch.int64
    if dtype.is_complex or x.dtype.is_complex:
        raise NotImplementedError("mi355 backend: complex reductions are not supported")
    if op == _lib.MEAN and not dtype.is_floating_point:
        raise RuntimeError(f"{name}(): could not infer output dtype. Optional dtype must be either a floating "
                           f"point or complex dtype. Got: {str(dtype).replace('torch.', '').capitalize()}")
    shape = _out_shape(x, dims, keepdim)
    red = prod(x.shape[d] for d in dims) if x.dim() else 1
    if x.numel() == 0:
        fill = float("nan") if (op == _lib.MEAN and red == 0) else 0
        return torch.full(shape, fill, dtype=dtype, device=x.device)
    # Pick the dtype the kernel reads (`src`) and writes (`native_out`); cast around it.
    if dtype.is_floating_point:
        src = x if x.dtype.is_floating_point else cast(x, dtype)
        if src.dtype != dtype and not (src.dtype in (torch.float16, torch.bfloat16) and dtype == torch.float32):
            src = cast(src, dtype)
        native_out = dtype
    else:
        src = cast(x, torch.int64) if x.dtype not in (torch.int32, torch.int64) else x
        native_out = torch.int64
    out = _run_reduce(op, src, dims, keepdim, native_out)
    return cast(out, dtype)


@device_managed
def sum_dim(self, dim=None, keepdim=False, *, dtype=None):
    """aten.sum.dim_IntList"""
    return _sum_like(_lib.SUM, self, dim, keepdim, dtype, "sum")


@device_managed
def sum_default(self, *, dtype=None):
    """aten.sum.default"""
    return _sum_like(_lib.SUM, self, None, False, dtype, "sum")


@device_managed
def mean_dim(self, dim=None, keepdim=False, *, dtype=None):
    """aten.mean.dim"""
    return _sum_like(_lib.MEAN, self, dim, keepdim, dtype, "mean")


@device_managed
def mean_default(self, *, dtype=None):
    """aten.mean.default"""
    return _sum_like(_lib.MEAN, self, None, False, dtype, "mean")


def _max_src(x):
    if x.dtype in _NATIVE_IN:
        return x
    if x.dtype in _SMALL_INT:
        return cast(x, torch.int32)  # value preserving
    raise NotImplementedError(f"mi355 backend: dtype {x.dtype} is not supported")


@device_managed
def amax(self, dim=(), keepdim=False):
    """aten.amax.default: NaN propagates; dim=[] reduces everything."""
    dims = _norm_dims(list(dim), self.dim())
    shape = _out_shape(self, dims, keepdim)
    for d in dims:
        if self.dim() and self.shape[d] == 0:
            raise IndexError(f"amax(): Expected reduction dim {d} to have non-zero size.")
    if self.numel() == 0:
        return new_dense(shape, self.dtype, self.device)
    src = _max_src(self)
    return cast(_run_reduce(_lib.AMAX, src, dims, keepdim, src.dtype), self.dtype)


@device_managed
def argmax(self, dim=None, keepdim=False):
    """aten.argmax.default: first index of the maximum, NaN counts as maximum."""
    if dim is None:
        if self.numel() == 0:
            raise IndexError("argmax(): Expected reduction dim to be specified for input.numel() == 0. Specify the reduction dim with the 'dim' argument.")
        flat = dense(self).view(-1)
        out = _run_reduce(_lib.ARGMAX, _max_src(flat), [0], False, torch.int64)
        return out.view([1] * self.dim()) if keepdim else out
    d = norm_dim(dim, self.dim())
    if self.dim() and self.shape[d] == 0:
        raise IndexError(f"argmax(): Expected reduction dim {d} to have non-zero size.")
    dims = [d] if self.dim() else []
    if self.numel() == 0:
        return new_dense(_out_shape(self, dims, keepdim), torch.int64, self.device)
    return _run_reduce(_lib.ARGMAX, _max_src(self), dims, keepdim, torch.int64)


def _softmax_impl(self, dim, half_to_float, log):
    if not self.dtype.is_floating_point:
        raise RuntimeError("softmax expects a floating point input")
    if half_to_float and self.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("conversion is supported for Half and BFloat16 type only")
    out_dtype = torch.float32 if half_to_float else self.dtype
    d = norm_dim(dim, self.dim())
    out = new_result(self.shape, out_dtype, self.device)
    if self.numel() == 0:
        return out
    x = dense(self)
    shape = x.shape if x.dim() else (1,)
    outer, n, inner = prod(shape[:d]), shape[d], prod(shape[d + 1 :])
    if (inner > 1 and n >= 256 and outer * ((inner + 63) // 64) < 256 and x.numel() >= 131072
            and x.dtype != torch.float64):
        # A long softmax axis over few columns gives the column kernels a handful of blocks that each
        # walk the axis serially.  Two tiled transposing copies around the row kernel are far
        # cheaper: [32, 1000, 49] fp32 takes 81 us on the column kernel and 26 us this way.
        rows = dense(x.view(outer, n, inner).transpose(1, 2))
        res = new_dense(rows.shape, out_dtype, self.device)
        launch("mi355_softmax", rows.data_ptr(), _lib.dtype_code(x.dtype), res.data_ptr(), _lib.dtype_code(out_dtype),
               outer * inner, n, 1, 1 if log else 0, None, 0)
        copy_into(out.view(outer, n, inner), res.transpose(1, 2))
        return out
    ws, ws_bytes = _row_workspace(outer, n, x) if inner == 1 else (None, 0)
    launch("mi355_softmax", x.data_ptr(), _lib.dtype_code(x.dtype), out.data_ptr(), _lib.dtype_code(out_dtype),
           outer, n, inner, 1 if log else 0, ws.data_ptr() if ws is not None else None, ws_bytes)
    return out


@device_managed
def softmax(self, dim, half_to_float):
    """aten._softmax.default"""
    return _softmax_impl(self, dim, half_to_float, False)


@device_managed
def log_softmax(self, dim, half_to_float):
    """aten._log_softmax.default"""
    return _softmax_impl(self, dim, half_to_float, True)


@device_managed
def native_layer_norm(input, normalized_shape, weight, bias, eps):
    """aten.native_layer_norm.default -> (y, mean, rstd).

    mean/rstd are fp32 for f16/bf16 inputs, fp64 for f64 (the accumulation type, as ATen's GPU kernels
    return them) and shaped input.shape[:-k] + [1]*k.
    """
    k = len(normalized_shape)
    if k == 0 or list(input.shape[input.dim() - k :]) != list(normalized_shape):
        raise RuntimeError(
            f"Given normalized_shape={list(normalized_shape)}, expected input with shape "
            f"[*, {', '.join(str(s) for s in normalized_shape)}], but got input of size{list(input.shape)}")
    for name, p in (("weight", weight), ("bias", bias)):
        if p is not None and list(p.shape) != list(normalized_shape):
            raise RuntimeError(f"Expected {name} to be of same shape as normalized_shape, but got {name} of shape "
                               f"{list(p.shape)} and normalized_shape = {list(normalized_shape)}")
    if input.dtype not in (torch.float32, torch.float16, torch.bfloat16, torch.float64):
        raise NotImplementedError(f"mi355 backend: layer norm on {input.dtype} is not supported")
    lead = list(input.shape[: input.dim() - k])
    M, N = prod(lead), prod(normalized_shape)
    stat_dtype = torch.float64 if input.dtype == torch.float64 else torch.float32
    y = new_result(input.shape, input.dtype, input.device)
    mean = new_result(lead + [1] * k, stat_dtype, input.device)
    rstd = new_result(lead + [1] * k, stat_dtype, input.device)
    if M == 0:
        return y, mean, rstd
    if N == 0:
        raise NotImplementedError("mi355 backend: layer norm over zero elements is not supported")
    w_dtype = None
    for p in (weight, bias):
        if p is not None:
            if w_dtype is not None and p.dtype != w_dtype:
                raise RuntimeError("weight and bias must have the same dtype")
            w_dtype = p.dtype
    if w_dtype is not None and w_dtype != input.dtype:
        if w_dtype != torch.float32 or input.dtype == torch.float64:
            weight = cast(weight, input.dtype) if weight is not None else None
            bias = cast(bias, input.dtype) if bias is not None else None
            w_dtype = input.dtype
    x = dense(input)
    w = dense(weight) if weight is not None else None
    b = dense(bias) if bias is not None else None
    ws, ws_bytes = _row_workspace(M, N, x)
    launch("mi355_layer_norm", x.data_ptr(), _lib.dtype_code(x.dtype), w.data_ptr() if w is not None else None,
           b.data_ptr() if b is not None else None, _lib.dtype_code(w_dtype or x.dtype), y.data_ptr(),
           mean.data_ptr(), rstd.data_ptr(), _lib.dtype_code(stat_dtype), M, N, float(eps),
           ws.data_ptr() if ws is not None else None, ws_bytes)
    return y, mean, rstd
