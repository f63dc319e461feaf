"""One canonical OpOverload object per spec name ("add.Tensor", "relu").

Mirror of BackendBench/opregistry.py:14-110: suites and backends key their tables by the
same object so that `op in backend` is an identity lookup.
"""

import torch


def spec_name(op):
    """"aten::add.Tensor" -> "add.Tensor"; None for objects that are not aten overloads."""
    full = getattr(op, "_name", None)
    if isinstance(full, str) and "::" in full:
        return full.split("::", 1)[1]
    return None


class OpRegistry:
    def __init__(self):
        self._ops = {}

    def get_operator(self, key):
        name = key if isinstance(key, str) else spec_name(key)
        if name is None:
            return key
        if name in self._ops:
            return self._ops[name]
        base, _, overload = name.partition(".")
        try:
            op = getattr(getattr(torch.ops.aten, base), overload or "default")
        except AttributeError:
            return None if isinstance(key, str) else key
        self._ops[name] = op
        return op

    def register_operator(self, op):
        name = spec_name(op)
        if name is not None:
            self._ops[name] = op

    def has_operator(self, name):
        return name in self._ops

    def clear(self):
        self._ops.clear()

    def __len__(self):
        return len(self._ops)

    def __contains__(self, name):
        return name in self._ops


_registry = OpRegistry()


def get_operator(key):
    return _registry.get_operator(key)


def register_operator(op):
    _registry.register_operator(op)


def get_registry():
    return _registry
