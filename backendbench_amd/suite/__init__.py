"""Test suites: containers, the reference's smoke suite, and this operator set's own suite."""

from .base import OpTest, Test, TestSuite
from .baseline import BaselineTestSuite, Case, edge_cases, out_perf_cases, perf_cases
from .smoke import SmokeTestSuite

__all__ = ["OpTest", "Test", "TestSuite", "SmokeTestSuite", "BaselineTestSuite", "Case", "edge_cases", "out_perf_cases", "perf_cases"]
