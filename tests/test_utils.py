"""Name plumbing, argument strings, error metrics and the stream scan.  The literal strings
and values are the ones the reference's own tests expect (test/test_utils.py:181-330,
336-453, 545-607, 24-173; docstrings of BackendBench/utils.py:296-300, 321-324)."""

import math

import pytest
import torch

from backendbench_amd.utils import (compute_errors, deserialize_args, folder_name_to_op_name, get_pytorch_op,
                                    is_overload_folder_name, op_name_to_folder_name, serialize_args,
                                    uses_cuda_stream)


@pytest.mark.parametrize("op,folder", [("add.Tensor", "add__Tensor"), ("nn.functional.relu", "nn__functional__relu"),
                                       ("aten.add.Tensor", "aten__add__Tensor"), ("_native_batch_norm", "_native_batch_norm"),
                                       ("add_.Tensor", "add___Tensor"), ("relu.default", "relu__default"),
                                       ("sum.dim_IntList", "sum__dim_IntList"), ("_softmax.default", "_softmax__default")])
def test_name_round_trip(op, folder):
    assert op_name_to_folder_name(op) == folder
    assert folder_name_to_op_name(folder) == op


def test_overload_folder_detection():
    assert is_overload_folder_name("add__Tensor") and is_overload_folder_name("nn__functional__relu")
    assert not is_overload_folder_name("add") and not is_overload_folder_name("_native_batch_norm")
    assert not is_overload_folder_name("my_op_name")


def test_get_pytorch_op():
    assert get_pytorch_op("add.Tensor") is torch.ops.aten.add.Tensor
    assert get_pytorch_op("relu.default") is torch.ops.aten.relu.default
    assert get_pytorch_op("relu") is torch.ops.aten.relu.default
    assert get_pytorch_op("add_.Tensor") is torch.ops.aten.add_.Tensor
    assert get_pytorch_op("no_such_op.default") is None
    assert get_pytorch_op("add.NoSuchOverload") is None


SERIALIZE_CASES = [
    (lambda: ([torch.empty(48, 24, 28, 28, dtype=torch.float16)], {}), "((T([48, 24, 28, 28], f16),), {})"),
    (lambda: ([torch.empty(8, 8, 8, 8, 8, dtype=torch.float16)] * 2, {}),
     "((T([8, 8, 8, 8, 8], f16), T([8, 8, 8, 8, 8], f16),), {})"),
    (lambda: ([], {}), "((), {})"),
    (lambda: ([1, 2.5, "hello", True, None], {}), "((1, 2.5, 'hello', True, None,), {})"),
    (lambda: ([[torch.empty(5, 5), torch.empty(3, 3, dtype=torch.int64), 42]], {}),
     "(([T([5, 5], f32), T([3, 3], i64), 42],), {})"),
    (lambda: ([], {"weight": torch.empty(3, 3), "bias": None, "alpha": 0.5}),
     "((), {'weight': T([3, 3], f32), 'bias': None, 'alpha': 0.5})"),
    (lambda: ([torch.empty(128, 256, dtype=torch.float16), [1024, 249, 249]],
              {"dtype": torch.float16, "layout": torch.strided, "device": "cpu"}),
     "((T([128, 256], f16), [1024, 249, 249],), {'dtype': torch.float16, 'layout': torch.strided, 'device': 'cpu'})"),
]


@pytest.mark.parametrize("make,expected", SERIALIZE_CASES)
def test_serialize_literal(make, expected):
    args, kwargs = make()
    assert serialize_args(args, kwargs) == expected


@pytest.mark.parametrize("dtype,abbr", [(torch.float32, "f32"), (torch.float64, "f64"), (torch.bfloat16, "bf16"),
                                        (torch.int32, "i32"), (torch.int64, "i64"), (torch.bool, "b8"),
                                        (torch.float16, "f16"), (torch.uint8, "u8"), (torch.int8, "i8")])
def test_serialize_dtypes(dtype, abbr):
    assert serialize_args([torch.empty(10, 20, dtype=dtype)], {}) == f"((T([10, 20], {abbr}),), {{}})"


def test_serialize_strided_and_none():
    t = torch.empty(400, dtype=torch.float16).as_strided((10, 20), (40, 2))
    assert serialize_args([t], {}) == "((T([10, 20], f16, [40, 2]),), {})"
    assert serialize_args(None, {}) == "None" and serialize_args([], None) == "None"


def test_deserialize_tensor_specs():
    args, kwargs = deserialize_args("((T([48, 24, 28, 28], f16),), {})")
    assert len(args) == 1 and kwargs == {} and args[0].shape == (48, 24, 28, 28) and args[0].dtype == torch.float16
    args, _ = deserialize_args("((T([10, 20], f16, [40, 2]),), {})")
    assert args[0].shape == (10, 20) and args[0].stride() == (40, 2)
    args, kwargs = deserialize_args("((T([5, 5], f32), 42,), {'alpha': 0.5, 'beta': T([3, 3], i64)})")
    assert args[1] == 42 and kwargs["alpha"] == 0.5 and kwargs["beta"].dtype == torch.int64
    args, kwargs = deserialize_args(
        "((T([128, 256], f16), [1024, 249, 249],), {'dtype': torch.float16, 'layout': torch.strided, 'device': 'cuda'})")
    assert args[1] == [1024, 249, 249] and kwargs == {"dtype": torch.float16, "layout": torch.strided, "device": "cuda"}
    for abbr, dt in [("f32", torch.float32), ("f64", torch.float64), ("bf16", torch.bfloat16), ("i32", torch.int32),
                     ("i64", torch.int64), ("b8", torch.bool)]:
        assert deserialize_args(f"((T([10, 20], {abbr}),), {{}})")[0][0].dtype == dt


def test_deserialize_primitives():
    assert deserialize_args("((), {})") == ((), {})
    args, _ = deserialize_args("((1, 2.5, 'hello', True, None,), {})")
    assert args == (1, 2.5, "hello", True, None)
    assert deserialize_args("((inf,), {})")[0][0] == math.inf
    assert deserialize_args("((torch.float16,), {})")[0][0] == torch.float16
    assert deserialize_args("((T([10, 20], f32), [-1, -2, -3],), {})")[0][1] == [-1, -2, -3]
    # 4-argument form with an explicit device (test/test_torchbench_suite.py:14-45)
    t = deserialize_args("((T([3, 4], f32, None, 'cpu'),), {})")[0][0]
    assert t.device.type == "cpu" and t.shape == (3, 4)


def test_deserialized_floats_are_unit_interval():
    t = deserialize_args("((T([64, 64], f32),), {})")[0][0]
    assert (t >= 0).all() and (t <= 1).all()


def test_round_trip_keeps_the_string():
    s = "((T([7, 3], bf16), T([3], bf16), 2,), {'alpha': 0.25})"
    args, kwargs = deserialize_args(s)
    assert serialize_args(list(args), kwargs) == s


def test_compute_errors_known_values():
    e = compute_errors(torch.tensor([1.0, 2, 3, 4]), torch.tensor([1.0, 2, 3, 4]))
    assert e == (0.0, 0.0)
    a, r = compute_errors(torch.tensor([2.0, 4, 6, 8]), torch.tensor([2.2, 4.4, 6.6, 8.8]))
    assert a == pytest.approx(0.8, rel=1e-5) and r == pytest.approx(0.1, rel=1e-5)
    a, r = compute_errors(torch.tensor([0.0, 1.0]), torch.tensor([0.1, 1.1]))
    assert a == pytest.approx(0.1, rel=1e-5) and r > 1e6  # division by eps at the zero reference
    assert compute_errors(torch.zeros(2), torch.zeros(3)) == (None, None)
    assert compute_errors(torch.zeros(0), torch.zeros(0)) == (0.0, 0.0)
    a, r = compute_errors([torch.tensor([1.0, 2.0]), torch.tensor([3.0, 4.0])],
                          [torch.tensor([1.1, 2.2]), torch.tensor([3.3, 4.4])])
    assert a == pytest.approx(0.4, rel=1e-5) and r == pytest.approx(0.1, rel=1e-4)
    assert compute_errors(1.0, 2.0) == (None, None) and compute_errors([1, 2], [1, 2]) == (None, None)
    assert compute_errors([torch.zeros(1)], [torch.zeros(1), torch.zeros(1)]) == (None, None)


def _uses_ctor():
    s = torch.cuda.Stream()
    return s


def _uses_lowercase():
    s = stream()  # noqa: F821
    return s


def _uses_factory():
    return make_stream()  # noqa: F821


def _clean(x):
    handle = torch.cuda.current_stream()  # querying the current stream is fine
    return x + 1, handle


def test_stream_scan():
    assert uses_cuda_stream(_uses_ctor) and uses_cuda_stream(_uses_lowercase) and uses_cuda_stream(_uses_factory)
    assert not uses_cuda_stream(_clean)
    assert not uses_cuda_stream(torch.ops.aten.relu.default)  # no source: clean
    assert not uses_cuda_stream(len)


def test_our_entry_points_pass_the_stream_scan(repo_root):
    from backendbench_amd.backends import DirectoryBackend
    import os

    backend = DirectoryBackend(os.path.join(repo_root, "generated_kernels"))
    assert len(backend.compiled_kernels) == 68
    for impl in backend.compiled_kernels.values():
        assert not uses_cuda_stream(impl)


def test_python_side_broadcasting_matches_torch():
    """The wrappers broadcast shapes and strides themselves (torch.broadcast_shapes and expand()
    cost more host time than a kernel launch): same results as torch on random shapes."""
    import random

    import torch

    from backendbench_amd import _lib
    from backendbench_amd.ops.elementwise import _broadcast_shape, _clamp_dtype, _desc_as

    rng = random.Random(0)
    for _ in range(300):
        full = [rng.choice([1, 2, 3, 5]) for _ in range(rng.randint(0, 4))]
        shapes = []
        for _ in range(rng.randint(2, 3)):
            s = [1 if rng.random() < 0.3 else v for v in full]
            shapes.append(s[rng.randint(0, len(s)):] if rng.random() < 0.4 else s)
        want = torch.broadcast_shapes(*shapes)
        assert _broadcast_shape(*[torch.Size(s) for s in shapes]) == want
        t = torch.empty(shapes[0])
        ours = _lib.TensorDesc.from_buffer_copy(_desc_as(t, want))
        ref = _lib.TensorDesc.from_buffer_copy(_lib.desc(t.expand(want)))
        assert (ours.data, ours.dtype, ours.ndim, list(ours.sizes)) == (ref.data, ref.dtype, ref.ndim, list(ref.sizes))
        for size, a, b in zip(ours.sizes, ours.strides, ref.strides):   # strides of size-1 dims never matter
            assert size <= 1 or a == b
    with pytest.raises(RuntimeError):
        _broadcast_shape(torch.Size([2, 3]), torch.Size([4, 3]))
    assert torch.broadcast_shapes((0, 3), (1, 3)) == _broadcast_shape(torch.Size([0, 3]), torch.Size([1, 3]))
    for dt in (torch.float32, torch.bfloat16, torch.int32, torch.int64, torch.uint8):
        for bounds in ((1, None), (None, 2.5), (0.5, 1), (1, 2)):
            t = torch.zeros(3, dtype=dt)
            assert _clamp_dtype(t, bounds) == torch.clamp(t, *bounds).dtype


def test_packed_descriptor_layout():
    import ctypes

    import torch

    from backendbench_amd import _lib

    t = torch.empty(4, 6, 8)[:, ::2, 1:]
    d = _lib.TensorDesc.from_buffer_copy(_lib.desc(t))
    assert d.data == t.data_ptr() and d.dtype == _lib.F32 and d.ndim == 3
    assert list(d.sizes)[:3] == [4, 3, 7] and list(d.strides)[:3] == [48, 16, 1]
    assert list(d.sizes)[3:] == [0] * 5 and ctypes.sizeof(d) == len(_lib.desc(t))
    with pytest.raises(NotImplementedError):
        _lib.desc(torch.empty(2, dtype=torch.complex64))
    with pytest.raises(NotImplementedError):
        _lib.desc(torch.empty([1] * 9))
