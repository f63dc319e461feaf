"""The identity backend (BackendBench/backends/aten.py:10-18): every op implements itself."""

from .base import Backend


class AtenBackend(Backend):
    def __init__(self):
        super().__init__("aten")

    def __contains__(self, op):
        return True

    def __getitem__(self, op):
        return op
