"""``mamtorch.nn.v4`` (mamtorch/nn/v4/__init__.py:1): the current layer."""
from .fullyconnected import *  # noqa: F401,F403
from .fullyconnected import __all__  # noqa: F401
