"""``FullyConnected`` is the MAM layer (mamtorch/nn/__init__.py:6 exports the v4 module)."""
from .fullyconnected import FullyConnected

__all__ = ["FullyConnected"]
