"""``mamtorch_kernel_sparsev1`` wrappers (mamtorch/sparse/kernel/v1/__init__.py:1-4); the native
library that registers the operators is loaded by the package root."""
from .cusparsemm import cusparsemm

__all__ = ["cusparsemm"]
