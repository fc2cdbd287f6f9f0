"""``mamtorch.nn.v1`` (mamtorch/nn/v1/__init__.py:1): the older layer under its reference name."""
from .fullyconnected import *  # noqa: F401,F403
from .fullyconnected import __all__  # noqa: F401
