"""Helpers shared by the operator wrappers: device management, dense/cast copies done
with our own copy kernel, and the sticky out-of-range flag of the indexing kernels.

The wrappers may run as the registered kernel of an ATen overload (torch.library
override), so they never call an operator this backend overrides; allocation and view
ops (empty, empty_like, empty_strided, expand, view, as_strided, to) are the only torch
calls on tensors.
"""

import functools
import ctypes
import os

import torch

from .. import _lib


def _is_gpu(t):
    return t.device.type == "cuda"


def device_managed(fn):
    """Run `fn` on the GPU whatever device the arguments live on.

    Mirrors the contract the reference gives kernel authors
    (BackendBench/prompts.py:18-24): CPU tensors are moved to the GPU, the result goes
    back to the device of the first tensor argument, and a missing GPU is an error.
    """

    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        first = None
        all_gpu = True
        for a in args:
            if isinstance(a, torch.Tensor):
                if first is None:
                    first = a
                if not a.is_cuda:
                    all_gpu = False
        if kwargs:
            for a in kwargs.values():
                if isinstance(a, torch.Tensor):
                    if first is None:
                        first = a
                    if not a.is_cuda:
                        all_gpu = False
        if all_gpu:
            return fn(*args, **kwargs)
        _lib.require_gpu()
        home = first.device
        target = None
        for a in list(args) + list(kwargs.values()):
            if isinstance(a, torch.Tensor) and _is_gpu(a):
                target = a.device
                break
        if target is None:
            target = torch.device("cuda", torch.cuda.current_device())

        def mv(a):
            return a.to(target) if isinstance(a, torch.Tensor) and not _is_gpu(a) else a

        out = fn(*[mv(a) for a in args], **{k: mv(v) for k, v in kwargs.items()})
        if home.type == "cuda":
            return out
        if isinstance(out, torch.Tensor):
            return out.to(home)
        return tuple(o.to(home) for o in out)

    return wrapper


_entry = {}
_ready = set()  # devices mi355_init() has accepted
_current_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def launch(name, *args):
    """Call one C entry point with the current stream appended; raise on failure."""
    for w in _flag_words:
        if w.value:
            poll_index_errors()
            break
    fn = _entry.get(name)
    if fn is None:
        fn = _entry[name] = getattr(_lib.load(), name)
    dev = _current_device()
    if dev not in _ready:
        _lib.init_device(dev)  # refuses a GPU the launch heuristics are not built for
        _ready.add(dev)
    rc = fn(*args, _lib.current_stream_handle())
    if rc != 0:
        _lib.check(rc)


def row_major_strides(shape):
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * max(shape[i + 1], 1)
    return strides


def new_dense(shape, dtype, device):
    """Uninitialised row-major tensor (empty_strided parses its arguments faster than empty)."""
    return torch.empty_strided(shape, row_major_strides(shape), dtype=dtype, device=device)


# ---- out= overloads write in place ---------------------------------------------------
# An out= overload offers its `out` tensor(s) here before it calls the functional wrapper; the
# wrapper asks for its result buffer with new_result() / result_like() and gets `out` itself when
# shape, dtype, device and layout are the ones it would have allocated.  The kernel then writes
# straight into `out`: no temporary, no second pass.  Anything else (a resize, a cast, an `out`
# that shares memory with an input) leaves the offer untaken and the overload copies as before.
_offered = []


def offer_out(*outs):
    _offered[:] = outs


def withdraw_out():
    _offered.clear()


def _take(shape, dtype, device, strides):
    for i, t in enumerate(_offered):
        if t.dtype == dtype and t.device == device and tuple(t.shape) == tuple(shape) and t.stride() == tuple(strides):
            return _offered.pop(i)
    return None


def new_result(shape, dtype, device):
    """Row-major buffer for an operator's result: the offered out= tensor when it fits, else a new one."""
    if _offered:
        t = _take(shape, dtype, device, row_major_strides(shape))
        if t is not None:
            return t
    return torch.empty_strided(shape, row_major_strides(shape), dtype=dtype, device=device)


def result_like(lead, dtype):
    """Result buffer with the (permuted-dense) layout of `lead`: the offered out= tensor when it has exactly
    that layout, else torch.empty_like's."""
    out = torch.empty_like(lead) if lead.dtype == dtype else torch.empty_like(lead, dtype=dtype)
    if _offered:
        t = _take(out.shape, dtype, out.device, out.stride())
        if t is not None:
            return t
    return out


def copy_into(dst, src):
    """dst[...] = src (cast + arbitrary strides) with the mi355_copy kernel."""
    if dst.numel() == 0:
        return dst
    launch("mi355_copy", _lib.desc(src), _lib.desc(dst))
    return dst


def cast(t, dtype):
    """`t` in `dtype`, layout preserved; no-op when the dtype already matches."""
    if t.dtype == dtype:
        return t
    _lib.dtype_code(t.dtype)
    _lib.dtype_code(dtype)
    return copy_into(torch.empty_like(t, dtype=dtype), t)


def dense(t):
    """Row-major contiguous version of `t` (itself if it already is)."""
    if t.is_contiguous():
        return t
    _lib.dtype_code(t.dtype)
    return copy_into(new_dense(t.shape, t.dtype, t.device), t)


def prod(xs):
    p = 1
    for x in xs:
        p *= x
    return p


def norm_dim(dim, ndim):
    """ATen dim wrapping (a 0-d tensor accepts -1 and 0)."""
    n = max(ndim, 1)
    if not -n <= dim < n:
        raise IndexError(f"Dimension out of range (expected to be in range of [{-n}, {n - 1}], but got {dim})")
    return dim + n if dim < 0 else dim


# ---- out-of-range indices ----------------------------------------------------------
# The indexing kernels never dereference a bad index; they zero the output there and store 1 into a
# sticky int32 flag.  The flag lives in pinned host memory (device-accessible at its host address), so
# the error surfaces the way a device-side assert of the stock kernels does - asynchronously, without a
# device sync and without anything enqueued behind the kernel:
#   * every later call of any operator of this backend reads the flag word (a plain host load); once a
#     kernel has set it, that call raises IndexError naming the earlier indexing call;
#   * check_index_errors() synchronises and raises at once (this repository's evaluator calls it
#     after every test; MI355_SYNC_INDEX_CHECK=1 makes every indexing call do so, which is the
#     CPU kernels' behaviour at the cost of a device sync per call).
# Nothing raises while the stream is being captured into a graph (the flag stays set).
# Which call raises is therefore a matter of timing, as with a device-side assert: the first launch of this
# backend that finds the word set - any operator, possibly an unrelated one, which is then not launched -
# raises for every out-of-range index met up to that point; the words are cleared behind a device sync.
_flags = {}       # device key -> pinned int32 tensor (kept alive)
_flag_words = []  # ctypes views of the same words, read on every launch


def index_error_flag(device):
    """Address of this device's flag word, as the kernels' err_flag argument."""
    key = device.index if device.index is not None else torch.cuda.current_device()
    f = _flags.get(key)
    if f is None:
        f = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        _flags[key] = f
        _flag_words.append(ctypes.c_int32.from_address(f.data_ptr()))
    return f


def sync_index_check():
    return os.environ.get("MI355_SYNC_INDEX_CHECK", "0") == "1"


def poll_index_errors():
    """Non-blocking: raise IndexError if an earlier indexing call of this backend met an out-of-range
    index and the device has run it.  Called at the start of every operator launch when a flag is set."""
    if torch.cuda.is_current_stream_capturing():
        return  # not in the middle of a graph capture; the flag stays set
    if not any(w.value for w in _flag_words):
        return
    # Everything enqueued so far runs to its end before the words are cleared: a second indexing kernel
    # that is still storing 1 cannot slip its error past the clear and have it reported against some later,
    # innocent call (the error path may cost a device sync; the check above does not).
    torch.cuda.synchronize()
    bad = False
    for w in _flag_words:
        if w.value != 0:
            bad = True
            w.value = 0
    if bad:
        raise IndexError("index out of range in self (met by an earlier index_select / embedding / gather call of "
                         "this backend, whose output was zero-filled at that index)")


def check_index_errors():
    """Synchronise and raise IndexError if any indexing kernel saw an out-of-range index since the last check."""
    if not _flag_words:
        return
    torch.cuda.synchronize()
    bad = False
    for w in _flag_words:
        if w.value != 0:
            bad = True
            w.value = 0
    if bad:
        raise IndexError("index out of range in self")
