"""Exact MAM forward with first-index argmax/argmin (mamtorch/kernel/v1/__init__.py:1-4)."""
from .fullyconnected import fullyconnected
