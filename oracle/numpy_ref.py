"""numpy float64 / exact-integer restatement of each operator's published definition
(test infrastructure, see oracle/__init__.py).  Used only to pin `aten_cpu`: small inputs,
no attention to speed.  Semantics follow the ATen operator documentation: schema strings
cited per function are those of `torch.ops.aten.<op>._schema`.
"""

import numpy as np


def add(a, b, alpha=1):
    """add.Tensor(Tensor self, Tensor other, *, Scalar alpha=1): self + alpha * other."""
    return a + alpha * b


def mul(a, b):
    """mul.Tensor(Tensor self, Tensor other)"""
    return a * b


def maximum(a, b):
    """maximum(Tensor self, Tensor other): elementwise max, NaN if either is NaN."""
    with np.errstate(invalid="ignore"):
        return np.where(np.isnan(a) | np.isnan(b), np.nan, np.where(a > b, a, b)) if a.dtype.kind == "f" else np.maximum(a, b)


def minimum(a, b):
    """minimum(Tensor self, Tensor other): elementwise min, NaN if either is NaN."""
    with np.errstate(invalid="ignore"):
        return np.where(np.isnan(a) | np.isnan(b), np.nan, np.where(a < b, a, b)) if a.dtype.kind == "f" else np.minimum(a, b)


def clamp_tensor(x, lo=None, hi=None):
    """clamp.Tensor(Tensor self, Tensor? min, Tensor? max): minimum(maximum(x, min), max)."""
    y = x
    if lo is not None:
        y = maximum(*np.broadcast_arrays(np.asarray(y, dtype=np.result_type(y, lo)), np.asarray(lo, dtype=np.result_type(y, lo))))
    if hi is not None:
        y = minimum(*np.broadcast_arrays(np.asarray(y, dtype=np.result_type(y, hi)), np.asarray(hi, dtype=np.result_type(y, hi))))
    return y


def log_softmax(x, dim):
    """_log_softmax: (x - max) - log(sum(exp(x - max))) along dim."""
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        m = np.max(x, axis=dim, keepdims=True)
        d = x - m
        return d - np.log(np.exp(d).sum(axis=dim, keepdims=True))


def relu(x):
    """relu(Tensor self): max(x, 0) with NaN kept."""
    with np.errstate(invalid="ignore"):
        return np.where(x <= 0, np.zeros_like(x), x)


def clamp(x, lo=None, hi=None):
    """clamp(Tensor self, Scalar? min, Scalar? max): min(max(x, lo), hi); NaN kept; a NaN
    bound makes every element NaN."""
    y = np.array(x, dtype=np.result_type(x, *(b for b in (lo, hi) if b is not None)), copy=True)
    nan = np.isnan(y) if y.dtype.kind == "f" else np.zeros(y.shape, bool)
    with np.errstate(invalid="ignore"):
        if lo is not None:
            y = np.where(y < lo, lo, y)
        if hi is not None:
            y = np.where(y > hi, hi, y)
    if y.dtype.kind == "f":
        y = np.where(nan, np.nan, y)
        for b in (lo, hi):
            if b is not None and isinstance(b, float) and np.isnan(b):
                y = np.full_like(y, np.nan)
    return y


def where(cond, a, b):
    """where.self(Tensor condition, Tensor self, Tensor other)"""
    return np.where(cond, a, b)


def _axes(dim, ndim):
    if dim is None or (isinstance(dim, (list, tuple)) and len(dim) == 0):
        return tuple(range(ndim))
    if isinstance(dim, int):
        dim = [dim]
    return tuple(d % max(ndim, 1) for d in dim)


def sum_(x, dim=None, keepdim=False):
    """sum.dim_IntList: integer and bool inputs accumulate in int64."""
    if x.dtype.kind in "iub":
        x = x.astype(np.int64)
    return x.sum(axis=_axes(dim, x.ndim), keepdims=keepdim)


def mean(x, dim=None, keepdim=False):
    """mean.dim: sum / count (NaN for an empty reduction)."""
    with np.errstate(invalid="ignore", divide="ignore"):
        ax = _axes(dim, x.ndim)
        count = np.prod([x.shape[a] for a in ax]) if x.ndim else 1
        return x.sum(axis=ax, keepdims=keepdim) / np.float64(count)


def amax(x, dim=(), keepdim=False):
    """amax: NaN-propagating maximum over dims ([] = all)."""
    return np.max(x, axis=_axes(list(dim), x.ndim), keepdims=keepdim)


def argmax(x, dim=None, keepdim=False):
    """argmax: index of the first maximum; NaN counts as the maximum; None flattens."""
    if dim is None:
        r = np.argmax(x.reshape(-1))
        return np.asarray(r).reshape([1] * x.ndim) if keepdim else np.asarray(r)
    r = np.argmax(x, axis=dim)
    return np.expand_dims(r, dim) if keepdim else r


def softmax(x, dim):
    """_softmax: exp(x - max) / sum(exp(x - max)) along dim."""
    with np.errstate(invalid="ignore", over="ignore"):
        m = np.max(x, axis=dim, keepdims=True)
        e = np.exp(x - m)
        return e / e.sum(axis=dim, keepdims=True)


def layer_norm(x, normalized_shape, weight=None, bias=None, eps=1e-5):
    """native_layer_norm -> (y, mean, rstd): biased variance over the trailing dims,
    rstd = 1 / sqrt(var + eps), stats keep the reduced dims as size 1."""
    k = len(normalized_shape)
    ax = tuple(range(x.ndim - k, x.ndim))
    mean_ = x.mean(axis=ax, keepdims=True)
    var = ((x - mean_) ** 2).mean(axis=ax, keepdims=True)
    rstd = 1.0 / np.sqrt(var + eps)
    y = (x - mean_) * rstd
    if weight is not None:
        y = y * weight
    if bias is not None:
        y = y + bias
    return y, mean_, rstd


def mm(a, b):
    """mm(Tensor self, Tensor mat2)"""
    return a @ b


def addmm(c, a, b, beta=1, alpha=1):
    """addmm: beta * self + alpha * (mat1 @ mat2); beta == 0 ignores self entirely."""
    prod = alpha * (a @ b)
    return prod if beta == 0 else beta * c + prod


def index_select(x, dim, index):
    """index_select: slices of x along dim in the order of index."""
    return np.take(x, np.asarray(index).reshape(-1), axis=dim)


def embedding(weight, indices):
    """embedding: weight[indices] with the index shape in front of the row."""
    out = np.empty(tuple(np.shape(indices)) + (weight.shape[1],), dtype=weight.dtype)
    flat = np.asarray(indices).reshape(-1)
    rows = out.reshape(-1, weight.shape[1])
    for j, i in enumerate(flat):  # plain loop on purpose: the definition itself
        rows[j] = weight[i]
    return out


def gather(x, dim, index):
    """gather: out[i][j][k] = x[index[i][j][k]][j][k] for dim 0, etc.; index may be smaller
    than x in the other dims."""
    out = np.empty(index.shape, dtype=x.dtype)
    for pos in np.ndindex(*index.shape):
        src = list(pos)
        src[dim] = index[pos]
        out[pos] = x[tuple(src)]
    return out
