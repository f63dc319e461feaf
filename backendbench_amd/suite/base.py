"""Test containers (BackendBench/suite/base.py:8-36).

A Test holds thunks; every access to `.args` / `.kwargs` calls them again, so a consumer
that wants both sides of a comparison to see the same tensors reads them once.
"""


class Test:
    __test__ = False  # not a pytest class

    def __init__(self, *args, **kwargs):
        self._args = args
        self._kwargs = kwargs

    @property
    def args(self):
        return [thunk() for thunk in self._args]

    @property
    def kwargs(self):
        return {k: thunk() for k, thunk in self._kwargs.items()}


class OpTest:
    def __init__(self, op, correctness_tests, performance_tests):
        self.op = op
        self.correctness_tests = correctness_tests
        self.performance_tests = performance_tests


class TestSuite:
    __test__ = False

    def __init__(self, name, optests):
        self.name = name
        self.optests = optests

    def __iter__(self):
        yield from self.optests
