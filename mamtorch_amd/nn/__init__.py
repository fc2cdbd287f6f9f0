"""``FullyConnected`` is the MAM layer (mamtorch/nn/__init__.py:6 exports the v4 module); ``convert``
holds the model-surgery helpers of the reference's ViT example; ``v1`` / ``v4`` are the reference's
sub-package names (mamtorch/nn/__init__.py:1-4)."""
from .fullyconnected import FullyConnected
from .convert import MAMMlp, add_mam_to_model, get_layers
from .legacy import FullyConnectedV1, MAMDense
from .conv import MAMConv1d, MAMConv2d
from . import compat, v1, v4

__all__ = ["FullyConnected", "MAMMlp", "add_mam_to_model", "get_layers", "FullyConnectedV1", "MAMDense", "MAMConv1d", "MAMConv2d", "compat", "v1", "v4"]
