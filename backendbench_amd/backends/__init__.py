"""Backends: objects mapping an ATen OpOverload to the callable that implements it."""

from .aten import AtenBackend
from .base import Backend
from .directory import DirectoryBackend

__all__ = ["Backend", "AtenBackend", "DirectoryBackend"]
