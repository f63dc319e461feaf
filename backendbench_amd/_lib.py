"""ctypes binding of libmi355_aten.so (declared in include/mi355_aten.h).

This is the only place that touches the C ABI.  There is no fallback: if the library has
not been built, or its ABI version differs, loading raises and every operator wrapper
fails with it.
"""

import ctypes
import struct
from ctypes import c_char_p, c_double, c_int, c_int32, c_int64, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libmi355_aten.so"
ABI_VERSION = 8
MAX_DIMS = 8

# mi355_dtype
F32, F16, BF16, F64, I32, I64, I16, I8, U8, BOOL = range(10)
DTYPE = {
    torch.float32: F32,
    torch.float16: F16,
    torch.bfloat16: BF16,
    torch.float64: F64,
    torch.int32: I32,
    torch.int64: I64,
    torch.int16: I16,
    torch.int8: I8,
    torch.uint8: U8,
    torch.bool: BOOL,
}
# mi355_binary_op / mi355_unary_op / mi355_reduce_op
ADD, MUL, MAXIMUM, MINIMUM = 0, 1, 2, 3
RELU, CLAMP = 0, 1
SUM, MEAN, AMAX, ARGMAX = 0, 1, 2, 3


class TensorDesc(ctypes.Structure):
    """struct mi355_tensor"""

    _fields_ = [
        ("data", c_void_p),
        ("dtype", c_int32),
        ("ndim", c_int32),
        ("sizes", c_int64 * MAX_DIMS),
        ("strides", c_int64 * MAX_DIMS),
    ]


# `const mi355_tensor*` arguments are passed as the 144 packed bytes of the struct (built by
# desc() with one struct.pack): several times cheaper per call than filling a ctypes Structure.
_P = c_char_p
_DESC = struct.Struct("=Qii8q8q")
assert _DESC.size == ctypes.sizeof(TensorDesc)
_PAD = (0,) * MAX_DIMS

# name -> (restype, argtypes); mirrors include/mi355_aten.h one to one.
SIGNATURES = {
    "mi355_abi_version": (c_int, []),
    "mi355_last_error": (c_char_p, []),
    "mi355_init": (c_int, []),
    "mi355_set_knob": (c_int, [c_char_p, c_char_p]),
    "mi355_binary": (c_int, [c_int, _P, _P, c_double, c_int64, _P, c_void_p]),
    "mi355_unary": (c_int, [c_int, _P, c_int, c_double, c_double, c_int64, c_int64, _P, c_void_p]),
    "mi355_where": (c_int, [_P, _P, _P, _P, c_void_p]),
    "mi355_clamp_tensor": (c_int, [_P, _P, _P, _P, c_void_p]),
    "mi355_copy": (c_int, [_P, _P, c_void_p]),
    "mi355_reduce_workspace_bytes": (c_int64, [c_int, c_int, c_int64, c_int64, c_int64]),
    "mi355_reduce": (
        c_int,
        [c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64, c_void_p],
    ),
    "mi355_reduce_static_max_bytes": (c_int64, []),
    "mi355_reduce_static": (
        c_int,
        [c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p],
    ),
    "mi355_row_workspace_bytes": (c_int64, [c_int64, c_int64, c_int]),
    "mi355_softmax": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p, c_int64,
                              c_void_p]),
    "mi355_layer_norm": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
         c_double, c_void_p, c_int64, c_void_p],
    ),
    "mi355_gemm_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int]),
    "mi355_gemm": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64,
         c_int64, c_int64, c_double, c_double, c_int, c_void_p, c_int64, c_void_p],
    ),
    "mi355_gemm_f32out": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64,
         c_int64, c_int64, c_double, c_double, c_int, c_void_p],
    ),
    "mi355_gemm_status": (c_int, []),
    "mi355_gemm_tile_columns": (c_int, [c_int64, c_int64, c_int64, ctypes.POINTER(c_int32), ctypes.POINTER(c_int32)]),
    "mi355_gemm_plan": (c_int, [c_int64, c_int64, c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_char_p, c_int64]),
    "mi355_calib_mfma": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355_index_select": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "mi355_gather": (c_int, [_P, c_int, _P, _P, c_void_p, c_void_p]),
}

_lib = None


def load():
    """dlopen the kernel library once; raise if it is missing or of another ABI."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP kernels first "
            "(python -m backendbench_amd._build); there is no fallback path"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.mi355_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libmi355_aten.so has ABI {got}, the Python side expects {ABI_VERSION}")
    _lib = lib
    return lib


_initialised = set()


def init_device(index):
    """mi355_init() once per device: refuses anything but a 256-CU gfx950 part and resolves the
    library's per-device addresses.  Called from the first launch on a device."""
    if index in _initialised:
        return
    rc = load().mi355_init()
    if rc != 0:
        check(rc)
    _initialised.add(index)


def set_knob(name, value=None):
    """Test / measurement hook: override (or, with None, restore) one of the library's knobs."""
    check(load().mi355_set_knob(name.encode(), None if value is None else str(value).encode()))


def check(rc):
    if rc != 0:
        msg = load().mi355_last_error()
        raise RuntimeError(f"mi355 kernel library error {rc}: {msg.decode() if msg else '?'}")


def dtype_code(dtype):
    try:
        return DTYPE[dtype]
    except KeyError:
        raise NotImplementedError(f"mi355 backend: dtype {dtype} is not supported") from None


def desc(t, sizes=None, strides=None):
    """Packed `struct mi355_tensor` for `t`, optionally viewed with other sizes/strides (elements)."""
    if sizes is None:
        sizes = t.shape
        strides = t.stride()
    nd = len(sizes)
    if nd > MAX_DIMS:
        raise NotImplementedError(f"mi355 backend: {nd}-d tensors exceed the {MAX_DIMS}-d limit")
    try:
        code = DTYPE[t.dtype]
    except KeyError:
        raise NotImplementedError(f"mi355 backend: dtype {t.dtype} is not supported") from None
    pad = _PAD[nd:]
    return _DESC.pack(t.data_ptr(), code, nd, *sizes, *pad, *strides, *pad)


try:  # raw hipStream_t of the current stream without building a torch.cuda.Stream object
    _raw_stream = torch._C._cuda_getCurrentRawStream
    _cur_device = torch._C._cuda_getDevice
except AttributeError:  # pragma: no cover - older/newer torch without these bindings
    _raw_stream = _cur_device = None


def current_stream_handle():
    """hipStream_t of torch's current stream, so callers' events bracket our kernels."""
    if _raw_stream is not None:
        return _raw_stream(_cur_device())
    return torch.cuda.current_stream().cuda_stream


def require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("mi355 backend: no GPU visible; these operators only run on an MI355X (HIP) device")
