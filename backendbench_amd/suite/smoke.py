"""Smoke suite (BackendBench/suite/smoke.py:18-35): relu on CPU tensors, randn(2) for
correctness and randn(1024, 1024) for timing."""

import torch

from ..opregistry import get_operator
from .base import OpTest, Test, TestSuite


def randn(*size, **kw):
    return lambda: torch.randn(*size, **kw)


SmokeTestSuite = TestSuite(
    "smoke",
    [
        OpTest(
            get_operator(torch.ops.aten.relu.default),
            [Test(randn(2, device="cpu"))],
            [Test(randn(2**10, 2**10, device="cpu"))],
        )
    ],
)
