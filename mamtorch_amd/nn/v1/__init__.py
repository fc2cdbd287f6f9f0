"""``mamtorch.nn.v1`` (mamtorch/nn/v1/__init__.py:1): the older layer under its reference name."""
from ..legacy import FullyConnectedV1 as FullyConnected

__all__ = ["FullyConnected"]
