"""``mamtorch.nn.v4.fullyconnected`` (mamtorch/nn/v4/fullyconnected.py:8-10): the current layer under its
reference module path."""
from ..fullyconnected import FullyConnected

__all__ = ["FullyConnected"]
