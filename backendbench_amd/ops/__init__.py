"""ATen-semantics wrappers over libmi355_aten.so, one callable per operator slot.

SLOTS maps the directory-backend folder name (BackendBench/utils.py:289-308 naming) to the
callable that fills `<folder>_kernel_impl`.
"""

from ._common import check_index_errors
from .elementwise import add, clamp, maximum, mul, relu, where
from .index import embedding, gather, index_select
from .matmul import addmm, mm
from .reduce import (amax, argmax, mean_default, mean_dim, native_layer_norm, softmax, sum_default, sum_dim)

SLOTS = {
    "add__Tensor": add,
    "mul__Tensor": mul,
    "maximum__default": maximum,
    "relu__default": relu,
    "clamp__default": clamp,
    "where__self": where,
    "sum__dim_IntList": sum_dim,
    "sum__default": sum_default,
    "mean__dim": mean_dim,
    "mean__default": mean_default,
    "amax__default": amax,
    "argmax__default": argmax,
    "_softmax__default": softmax,
    "native_layer_norm__default": native_layer_norm,
    "mm__default": mm,
    "addmm__default": addmm,
    "index_select__default": index_select,
    "embedding__default": embedding,
    "gather__default": gather,
}

__all__ = ["SLOTS", "check_index_errors", *sorted(f.__name__ for f in SLOTS.values())]
