"""Directory backend: implementations discovered on disk.

Same contract as BackendBench/backends/directory.py:18-110:
``<ops_dir>/<folder>/<folder>_implementation*.py`` (first file in sorted order) must define
``<folder>_kernel_impl``; ``<folder>`` is the overload name with "." written "__"; the
callable is registered for exactly that overload.  A folder that fails to load is logged
and skipped, it never aborts the scan.
"""

import importlib.util
import logging
import os

from ..utils import folder_name_to_op_name, get_pytorch_op
from .base import Backend

logger = logging.getLogger(__name__)


class DirectoryBackend(Backend):
    def __init__(self, ops_dir="generated_kernels"):
        super().__init__("directory")
        self.ops_dir = ops_dir
        self.compiled_kernels = {}
        self._scan()

    def _scan(self):
        if not os.path.exists(self.ops_dir):
            logger.warning("ops directory %s does not exist", self.ops_dir)
            return
        for folder in os.listdir(self.ops_dir):
            path = os.path.join(self.ops_dir, folder)
            if not os.path.isdir(path):
                continue
            prefix = f"{folder}_implementation"
            candidates = sorted(f for f in os.listdir(path) if f.startswith(prefix) and f.endswith(".py"))
            if not candidates:
                logger.debug("no implementation file in %s", path)
                continue
            op_name = folder_name_to_op_name(folder)
            try:
                impl = self._load(os.path.join(path, candidates[0]), folder)
                op = get_pytorch_op(op_name)
                if op is None:
                    logger.warning("no aten operator named %s (folder %s)", op_name, folder)
                    continue
                self.compiled_kernels[op] = impl
                logger.info("loaded %s from %s", op_name, candidates[0])
            except Exception as exc:  # a broken folder only drops its own op
                logger.error("could not load %s from %s: %s", op_name, candidates[0], exc)
        logger.info("DirectoryBackend: %d kernels from %s/", len(self.compiled_kernels), self.ops_dir)

    @staticmethod
    def _load(file_path, folder):
        """Execute the file as module `op_<folder>` (outside sys.modules) and return its entry point."""
        spec = importlib.util.spec_from_file_location(f"op_{folder}", file_path)
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
        name = f"{folder}_kernel_impl"
        if not hasattr(module, name):
            raise ValueError(f"No function named {name} found in {file_path}")
        return getattr(module, name)

    def __contains__(self, op):
        return op in self.compiled_kernels

    def __getitem__(self, op):
        try:
            return self.compiled_kernels[op]
        except KeyError:
            raise KeyError(
                f"Operator {op} not implemented in DirectoryBackend - add implementation to {self.ops_dir}/"
            ) from None
