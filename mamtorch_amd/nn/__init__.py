"""``FullyConnected`` is the MAM layer (mamtorch/nn/__init__.py:6 exports the v4 module); ``convert``
holds the model-surgery helpers of the reference's ViT example."""
from .fullyconnected import FullyConnected
from .convert import MAMMlp, add_mam_to_model, get_layers

__all__ = ["FullyConnected", "MAMMlp", "add_mam_to_model", "get_layers"]
