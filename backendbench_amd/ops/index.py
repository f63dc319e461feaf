"""index_select / embedding / gather on the HIP gather kernels (bit-exact copies)."""

import torch

from .. import _lib
from ._common import (check_index_errors, dense, device_managed, index_error_flag, launch, new_dense, new_result, norm_dim, prod,
                      sync_index_check)


def _rows(src, outer, n_src, inner, index, out):
    flag = index_error_flag(src.device)
    launch("mi355_index_select", src.data_ptr(), src.element_size(), outer, n_src, inner, index.data_ptr(),
           _lib.dtype_code(index.dtype), index.numel(), out.data_ptr(), flag.data_ptr())
    if sync_index_check():
        check_index_errors()


def _check_index(index, name):
    if index.dtype not in (torch.int32, torch.int64):
        raise RuntimeError(f"{name}(): Expected dtype int32 or int64 for index")


@device_managed
def index_select(self, dim, index):
    """aten.index_select.default"""
    _check_index(index, "index_select")
    if index.dim() > 1:
        raise IndexError("index_select(): Index is supposed to be a vector")
    d = norm_dim(dim, self.dim())
    _lib.dtype_code(self.dtype)
    if self.dim() == 0:
        if index.numel() != 1:
            raise IndexError("index_select(): Index to scalar can have only 1 value")
        shape, out_shape = (1,), ()
    else:
        shape = tuple(self.shape)
        out_shape = shape[:d] + (index.numel(),) + shape[d + 1 :]
    out = new_result(out_shape, self.dtype, self.device)
    if out.numel() == 0:
        return out
    _rows(dense(self), prod(shape[:d]), shape[d], prod(shape[d + 1 :]), dense(index), out)
    return out


@device_managed
def embedding(weight, indices, padding_idx=-1, scale_grad_by_freq=False, sparse=False):
    """aten.embedding.default: rows of `weight`; the trailing arguments only matter for backward."""
    _check_index(indices, "embedding")
    if weight.dim() != 2:
        raise RuntimeError("'weight' must be 2-D")
    _lib.dtype_code(weight.dtype)
    out = new_result(tuple(indices.shape) + (weight.shape[1],), weight.dtype, weight.device)
    if out.numel() == 0:
        return out
    _rows(dense(weight), 1, weight.shape[0], weight.shape[1], dense(indices), out)
    return out


@device_managed
def gather(self, dim, index, *, sparse_grad=False):
    """aten.gather.default: out[i][j][k] = self[i][index[i][j][k]][k] for dim == 1."""
    if index.dtype != torch.int64:
        raise RuntimeError("gather(): Expected dtype int64 for index")
    _lib.dtype_code(self.dtype)
    d = norm_dim(dim, self.dim())
    out = new_result(index.shape, self.dtype, self.device)
    if index.numel() == 0:
        return out
    # 0-d operands behave as one-element vectors
    src = self.view(1) if self.dim() == 0 else self
    idx = index.view(1) if index.dim() == 0 else index
    res = out.view(1) if out.dim() == 0 else out
    if src.dim() != idx.dim():
        raise RuntimeError("Index tensor must have the same number of dimensions as input tensor")
    for k in range(src.dim()):
        if k != d and idx.shape[k] > src.shape[k]:
            raise RuntimeError(f"Size does not match at dimension {k} expected index {list(idx.shape)} to be "
                               f"smaller than self {list(src.shape)} apart from dimension {d}")
    flag = index_error_flag(self.device)
    launch("mi355_gather", _lib.desc(src), d, _lib.desc(idx), _lib.desc(res), flag.data_ptr())
    if sync_index_check():
        check_index_errors()
    return out
