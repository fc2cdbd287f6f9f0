"""``mamtorch.nn.compat`` (mamtorch/nn/compat.py:6-8): the deprecated ``MAMDense`` layer under the module
path the reference star-imports into its package root."""
from .legacy import MAMDense

__all__ = ["MAMDense"]
