"""Operator wrappers of the sparse module, laid out as mamtorch/sparse/kernel/__init__.py:1."""
from . import v1

__all__ = ["v1"]
