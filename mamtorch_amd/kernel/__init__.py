"""Operator wrappers; same sub-packages as mamtorch/kernel/__init__.py:1-4 (v1 exact, v4 default)."""
from . import v1
from . import v4
