"""MI355X-native operator backend behind BackendBench's directory-backend boundary.

`enable()` / `disable()` / `BackendBench.enable(...)` install the kernels of a directory
backend into the live PyTorch dispatcher, with the interface of
BackendBench/__init__.py:29-158: one torch.library IMPL registration per loaded
overload, for the "CUDA" key (which is also the key of HIP devices) or "CPU"; dropping
the Library object removes the registrations again.
"""

import logging
from pathlib import Path

import torch

__version__ = "0.1.0"
__all__ = ["enable", "disable", "BackendBench"]

logger = logging.getLogger(__name__)

_library = None  # the torch.library.Library that enable() without `lib` registers into


def _register(lib, kernels, namespace="aten", dispatch_key="CUDA"):
    """lib.impl("<op>.<overload>", fn, key) for every {OpOverload: fn} entry."""
    assert dispatch_key in ["CPU", "CUDA"], "Only CPU and CUDA dispatch keys are supported"
    count = 0
    for op, impl in kernels.items():
        try:
            schema = op._schema
            name = f"{schema.name}.{schema.overload_name}" if schema.overload_name else schema.name
            lib.impl(name, impl, dispatch_key)
            count += 1
        except Exception as exc:  # some operators cannot be overridden
            logger.warning("Could not register %s: %s", op, exc)
    print(f"Successfully registered {count} custom operators" if count else "No custom operators registered")


def enable(kernel_dir=None, namespace="aten", dispatch_key="CUDA", lib=None):
    """Route the operators found in `kernel_dir` (default: ./generated_kernels next to the
    package) to their directory-backend implementations."""
    from .backends.directory import DirectoryBackend

    print("Enabling DirectoryBackend")
    kernel_dir = Path(kernel_dir) if kernel_dir is not None else Path(__file__).parents[1] / "generated_kernels"
    if not kernel_dir.exists():
        logger.warning("Kernel directory %s does not exist.", kernel_dir)
        return
    try:
        backend = DirectoryBackend(str(kernel_dir))
        if lib is None:
            global _library
            if _library is None:
                _library = torch.library.Library(namespace, "IMPL", dispatch_key)
            lib = _library
        _register(lib, backend.compiled_kernels, namespace, dispatch_key)
    except Exception as exc:
        logger.warning("Failed to enable DirectoryBackend: %s", exc)


def disable():
    """Drop the registrations made by enable(); ATen's own kernels are back afterwards."""
    global _library
    if _library is None:
        logger.warning("DirectoryBackend is not currently enabled")
        return
    _library = None
    print("DirectoryBackend disabled")


class _Context:
    """`with BackendBench.enable(dir):` — registrations live in a Library owned by the
    context and vanish with it on exit."""

    def __init__(self, kernel_dir=None, namespace="aten", dispatch_key="CUDA"):
        self.kernel_dir = kernel_dir
        self.namespace = namespace
        self.dispatch_key = dispatch_key
        self.lib = torch.library.Library(namespace, "IMPL", dispatch_key)

    def __enter__(self):
        enable(self.kernel_dir, self.namespace, self.dispatch_key, self.lib)
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        self.lib = None


class BackendBench:
    @classmethod
    def enable(cls, kernel_dir=None, namespace="aten", dispatch_key="CUDA"):
        return _Context(kernel_dir, namespace, dispatch_key)
