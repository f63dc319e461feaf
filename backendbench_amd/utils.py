"""Name plumbing, test-argument strings, error metrics and the stream scan.

Host-side mirror of the parts of BackendBench/utils.py the directory-backend path uses:
folder <-> operator names (utils.py:289-345), operator lookup (:252-278), the
`T([shape], dtype[, stride])` argument grammar (:100-182), max abs/rel error (:185-242)
and the static "does this implementation create streams" check (:50-97).
"""

import ast
import inspect
import math
import re
import textwrap

import torch
from torch.testing import make_tensor

ESCAPE = "__"  # stands for "." in folder names

DTYPE_ABBR = {
    torch.bfloat16: "bf16", torch.float64: "f64", torch.float32: "f32", torch.float16: "f16",
    torch.complex32: "c32", torch.complex64: "c64", torch.complex128: "c128",
    torch.int8: "i8", torch.int16: "i16", torch.int32: "i32", torch.int64: "i64",
    torch.bool: "b8", torch.uint8: "u8",
}
ABBR_DTYPE = {v: k for k, v in DTYPE_ABBR.items()}
_FLOATS = (torch.float16, torch.bfloat16, torch.float32, torch.float64)


# ---- names ---------------------------------------------------------------------------
def op_name_to_folder_name(op_name: str) -> str:
    """"add.Tensor" -> "add__Tensor"; names without a dot are unchanged."""
    return op_name.replace(".", ESCAPE)


def folder_name_to_op_name(folder: str) -> str:
    """"add__Tensor" -> "add.Tensor", and "add___Tensor" -> "add_.Tensor": the escape is
    matched from the right so an in-place op keeps its trailing underscore."""
    out = []
    i = len(folder)
    while i > 0:
        if i >= 2 and folder[i - 2 : i] == ESCAPE:
            out.append(".")
            i -= 2
        else:
            out.append(folder[i - 1])
            i -= 1
    return "".join(reversed(out))


def is_overload_folder_name(folder: str) -> bool:
    return ESCAPE in folder


def extract_operator_name(op_str: str) -> str:
    return op_str.split("aten.")[-1] if "aten." in op_str else op_str


def get_pytorch_op(op_name: str):
    """torch.ops.aten overload for "add.Tensor" / "relu.default" / "relu"; None if unknown."""
    base, _, overload = op_name.partition(".")
    try:
        return getattr(getattr(torch.ops.aten, base), overload or "default")
    except AttributeError:
        return None


# ---- argument strings ------------------------------------------------------------------
def _tensor_from_spec(size, dtype, stride=None, device="cuda"):
    """Random tensor of a serialized spec: floats uniform in [0, 1), strided specs as views."""
    kw = {"low": 0, "high": 1} if dtype in _FLOATS else {}
    if device == "cuda" and not torch.cuda.is_available():
        device = "cpu"
    if stride is None:
        return make_tensor(size, dtype=dtype, device=device, **kw)
    extent = 1 + sum((n - 1) * s for n, s in zip(size, stride))
    return make_tensor(extent, dtype=dtype, device=device, **kw).as_strided(size, stride)


def _ser(value):
    if isinstance(value, torch.Tensor):
        head = f"T({list(value.shape)}, {DTYPE_ABBR[value.dtype]}"
        return head + (")" if value.is_contiguous() else f", {list(value.stride())})")
    if isinstance(value, list):
        return "[" + ", ".join(_ser(v) for v in value) + "]"
    return repr(value)


def serialize_args(args, kwargs) -> str:
    """((arg, ...,), {'key': value, ...}) with tensors written as T([shape], dtype[, stride])."""
    if args is None or kwargs is None:
        return "None"
    pos = ", ".join(_ser(a) for a in args)
    kw = ", ".join(f"'{k}': {_ser(v)}" for k, v in kwargs.items())
    args_part = f"({pos},)" if pos else "()"
    return f"({args_part}, {{{kw}}})"


def deserialize_args(text):
    """Inverse of serialize_args: returns (args, kwargs) with freshly drawn tensors."""
    text = text.strip().strip("'")
    for abbr in ABBR_DTYPE:
        text = text.replace(f"'{abbr}'", abbr)
    text = re.sub(r'["\']torch\.device\((.*?)\)["\']', r"torch.device(\1)", text)
    env = {"T": _tensor_from_spec, "th": torch, "torch": torch, "inf": math.inf, **ABBR_DTYPE}
    return eval(text.strip().strip("'").strip('"'), env)


# ---- error metrics ---------------------------------------------------------------------
def compute_errors(ref, res, eps=1e-10):
    """(max abs error, max rel error) over tensors or (nested) sequences of tensors;
    (None, None) when the pair cannot be compared numerically."""
    if isinstance(ref, torch.Tensor) and isinstance(res, torch.Tensor):
        if ref.shape != res.shape or (ref.is_sparse and res.is_sparse):
            return None, None
        if ref.numel() == 0 and res.numel() == 0:
            return 0.0, 0.0
        a, b = ref.float(), res.float().to(ref.device)
        diff = (a - b).abs()
        return diff.max().item(), (diff / (a.abs() + eps)).max().item()
    if isinstance(ref, (list, tuple)) and isinstance(res, (list, tuple)):
        if len(ref) != len(res):
            return None, None
        if not any(isinstance(x, torch.Tensor) for x in ref) or not any(isinstance(x, torch.Tensor) for x in res):
            return None, None
        worst_abs = worst_rel = -math.inf
        for r, s in zip(ref, res):
            e_abs, e_rel = compute_errors(r, s)
            if e_abs is None or e_rel is None:
                continue
            worst_abs, worst_rel = max(worst_abs, e_abs), max(worst_rel, e_rel)
        return (None, None) if worst_abs == -math.inf else (worst_abs, worst_rel)
    return None, None


# ---- stream scan -----------------------------------------------------------------------
_STREAM_PATTERNS = [
    r"torch\.cuda\.Stream\(", r"cupy\.cuda\.Stream\(", r"cuda\.Stream\(", r"pycuda.*Stream\(",
    r"\bStream\(", r"make_stream\(", r"create_stream\(",
]


def uses_cuda_stream(func) -> bool:
    """True if the source of `func` constructs a stream (work on a side stream escapes the
    event timing).  Callables without retrievable or parsable source count as clean."""
    try:
        source = inspect.getsource(func)
        tree = ast.parse(textwrap.dedent(source))
    except (TypeError, OSError, IndentationError, SyntaxError):
        return False
    if any(re.search(p, source, re.IGNORECASE) for p in _STREAM_PATTERNS):
        return True
    for node in ast.walk(tree):
        if isinstance(node, ast.Call):
            f = node.func
            if getattr(f, "attr", None) == "Stream" or getattr(f, "id", None) == "Stream":
                return True
    return False
