import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def repo_root():
    return ROOT


class _GemmKnobs:
    """The library's GEMM test knobs (mi355_set_knob): a test forces one kernel form on a shape of its
    choosing; every knob a test touched is restored when the test ends."""

    def __init__(self):
        from backendbench_amd import _lib

        self._lib = _lib
        self._touched = set()

    def _set(self, name, value):
        self._touched.add(name)
        self._lib.set_knob(name, value)

    def tile(self, value):
        self._set("gemm_tile", value)

    def waves(self, value):
        self._set("gemm_waves", value)

    def split(self, value):
        self._set("gemm_split", value)

    def spin_limit(self, value):
        self._set("x16_spin_limit", value)

    def prefetch(self, value):
        self._set("gemm_prefetch", value)

    def restore(self):
        for name in self._touched:
            self._lib.set_knob(name, None)
        self._touched.clear()


@pytest.fixture
def gemm_knobs():
    knobs = _GemmKnobs()
    yield knobs
    knobs.restore()
