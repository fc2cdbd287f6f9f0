"""``mamtorch.nn.v1.fullyconnected`` (mamtorch/nn/v1/fullyconnected.py:6-8): the older layer under its
reference module path and class name."""
from ..legacy import FullyConnectedV1 as FullyConnected

__all__ = ["FullyConnected"]
