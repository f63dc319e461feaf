"""Replays operator traces: text files in the reference's TorchBench trace format.

    Operator: aten.add.Tensor
    cnt: 12, ((T([64, 128], bf16), T([128], bf16)), {})

(BackendBench/data_loaders.py:43-91 parses it, BackendBench/suite/torchbench.py:39-105
turns it into tests.)  Each `cnt:` line is one input of the operator named by the last
`Operator:` line; tensors are re-drawn from the spec on every use.  Inputs of an op are
ordered by decreasing byte size and may be cut to the `topn` largest.
"""

import re

import torch

from ..utils import deserialize_args


def args_size(args):
    total = 0
    for a in args:
        if isinstance(a, torch.Tensor):
            total += a.numel() * a.element_size()
        elif isinstance(a, (tuple, list)):
            total += args_size(a)
    return total


def parse_trace(lines, filter=None):
    """[{op_name, args, count}] from the lines of a trace."""
    entries, op = [], None
    for line in lines:
        if isinstance(line, bytes):
            line = line.decode()
        m = re.match(r"Operator: (.*)", line)
        if m:
            op = m.group(1).strip()
            if op == "aten.sum.SymInt":  # name used by older traces
                op = "aten.sum.dim_IntList"
            continue
        m = re.match(r"cnt: (\d+), (.*)", line)
        if m:
            assert op is not None, "cnt line before any Operator line"
            if filter is None or any(f in op for f in filter):
                entries.append({"op_name": op, "args": m.group(2), "count": int(m.group(1))})
    return entries


class TraceTest:
    def __init__(self, *args, **kwargs):
        self.args = args
        self.kwargs = kwargs


class TraceOpTest:
    def __init__(self, op, inputs, topn=None):
        obj = torch.ops
        for part in op.split("."):
            obj = getattr(obj, part)
        self.op = obj
        self.inputs = inputs
        self.topn = topn

    def tests(self):
        sized = []
        for text in self.inputs:
            args, kwargs = deserialize_args(text)
            sized.append((args_size(args) + args_size(list(kwargs.values())), text))
        ordered = [t for _, t in sorted(sized, reverse=True)]
        return ordered if self.topn is None else ordered[: self.topn]

    def _make(self):
        for text in self.tests():
            args, kwargs = deserialize_args(text)
            yield TraceTest(*args, **kwargs)

    @property
    def correctness_tests(self):
        return self._make()

    @property
    def performance_tests(self):
        return self._make()


class TraceTestSuite:
    def __init__(self, name, filename, filter=None, topn=None):
        self.name = name
        self.topn = topn
        with open(filename) as f:
            entries = parse_trace(f, filter)
        self.optests = {}
        for e in entries:
            bucket = self.optests.setdefault(e["op_name"], [])
            if e["args"] not in bucket:
                bucket.append(e["args"])

    def __iter__(self):
        for op, inputs in self.optests.items():
            yield TraceOpTest(op, inputs, self.topn)
