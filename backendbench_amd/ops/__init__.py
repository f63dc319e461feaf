"""ATen-semantics wrappers over libmi355_aten.so, one callable per operator slot.

SLOTS maps the directory-backend folder name (BackendBench/utils.py:289-308 naming) to the
callable that fills `<folder>_kernel_impl`.  CORE_SLOTS are the 19 overloads of the core
operator set; VARIANT_SLOTS are their in-place / out= / sibling overloads
(BackendBench/scripts/op_map.py lists them on the same `canonical:` lines), served by the
same kernels.
"""

from ._common import check_index_errors
from .elementwise import (_inplace_from, add, add_, clamp, clamp_, clamp_max, clamp_max_, clamp_max_tensor, clamp_min,
                          clamp_min_, clamp_min_tensor, clamp_tensor, maximum, minimum, mul, mul_, out_variant, relu,
                          relu_, tuple_out_variant, where)
from .index import embedding, gather, index_select
from .matmul import addmm, addmm_dtype, mm, mm_dtype
from .reduce import (amax, argmax, log_softmax, mean_default, mean_dim, native_layer_norm, softmax, sum_default,
                     sum_dim)

CORE_SLOTS = {
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

VARIANT_SLOTS = {
    # in-place overloads (folder names keep the trailing underscore: add_.Tensor -> add___Tensor)
    "add___Tensor": add_,
    "mul___Tensor": mul_,
    "relu___default": relu_,
    "clamp___default": clamp_,
    "add___Scalar": add_,
    "mul___Scalar": mul_,
    "clamp_min___default": clamp_min_,
    "clamp_max___default": clamp_max_,
    "clamp___Tensor": _inplace_from(clamp_tensor, "clamp_tensor_"),
    "addmm___default": _inplace_from(addmm, "addmm_"),
    # sibling overloads on the same kernels
    "minimum__default": minimum,
    "clamp_min__default": clamp_min,
    "clamp_max__default": clamp_max,
    "clamp__Tensor": clamp_tensor,
    "_log_softmax__default": log_softmax,
    "add__Scalar": add,   # a Python scalar takes the same promotion as a 0-d wrapped number
    "mul__Scalar": mul,
    "clamp_min__Tensor": clamp_min_tensor,
    "clamp_max__Tensor": clamp_max_tensor,
    "mm__dtype": mm_dtype,        # bf16 / f16 operands, fp32 result (BackendBench/scripts/op_map.py:740)
    "addmm__dtype": addmm_dtype,  # (op_map.py:271)
    # out= overloads
    "add__out": out_variant(add),
    "mul__out": out_variant(mul),
    "maximum__out": out_variant(maximum),
    "relu__out": out_variant(relu),
    "clamp__out": out_variant(clamp),
    "where__self_out": out_variant(where),
    "sum__IntList_out": out_variant(sum_dim),
    "mean__out": out_variant(mean_dim),
    "amax__out": out_variant(amax),
    "argmax__out": out_variant(argmax),
    "_softmax__out": out_variant(softmax),
    "mm__out": out_variant(mm),
    "addmm__out": out_variant(addmm),
    "index_select__out": out_variant(index_select),
    "gather__out": out_variant(gather),
    "add__Scalar_out": out_variant(add),
    "mul__Scalar_out": out_variant(mul),
    "minimum__out": out_variant(minimum),
    "clamp__Tensor_out": out_variant(clamp_tensor),
    "clamp_min__out": out_variant(clamp_min),
    "clamp_max__out": out_variant(clamp_max),
    "_log_softmax__out": out_variant(log_softmax),
    "sum__out": out_variant(sum_default),
    "mean__dtype_out": out_variant(mean_default),
    "embedding__out": out_variant(embedding),
    "native_layer_norm__out": tuple_out_variant(native_layer_norm, 3),
    "mm__dtype_out": out_variant(mm_dtype),
    "addmm__dtype_out": out_variant(addmm_dtype),
}

SLOTS = {**CORE_SLOTS, **VARIANT_SLOTS}

__all__ = ["SLOTS", "CORE_SLOTS", "VARIANT_SLOTS", "check_index_errors"]
