"""``mamtorch.nn.v4`` (mamtorch/nn/v4/__init__.py:1): the current layer."""
from ..fullyconnected import FullyConnected

__all__ = ["FullyConnected"]
