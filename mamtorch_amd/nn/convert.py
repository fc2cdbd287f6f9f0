"""Swapping ``nn.Linear`` layers of an existing model for MAM ``FullyConnected`` layers.

The reference does this for the MLP blocks of a ViT-B/16 in its ImageNet example
(examples/vitb16_imagenet1k/utils.py:50-77: ``get_layers`` resolves dotted paths, ``add_mam_to_ViT``
builds a ``FullyConnected`` of the same shape and moves weight and bias over).  The same two steps here,
for any module tree; ``MAMMlp`` is the block those paths name in a ViT (LayerNorm -> FC 768->3072 -> GELU
-> FC 3072->768), for use without the HuggingFace model around it.
"""
import torch
from torch import nn

from .fullyconnected import FullyConnected

__all__ = ["get_layers", "add_mam_to_model", "MAMMlp"]


def get_layers(model: nn.Module, layers_str, split_attributes: bool = False):
    """Modules at the dotted paths ``layers_str`` (examples/vitb16_imagenet1k/utils.py:50-65).  With
    ``split_attributes`` the parents and the last path components are returned apart."""
    paths = [layer.split('.') for layer in layers_str]
    attributes = [p[-1] for p in paths]
    if split_attributes:
        paths = [p[:-1] for p in paths]
    found = []
    for path in paths:
        module = model
        for name in path:
            module = getattr(module, name)
        found.append(module)
    return (found, attributes) if split_attributes else found


def add_mam_to_model(model: nn.Module, layers_str, vcon_steps: int = 0, layer_splits: int = 1,
                     vcon_type: str = 'linear', train_mam_only: bool = False, **fc_kwargs) -> nn.Module:
    """Replaces every ``nn.Linear`` named in ``layers_str`` by a ``FullyConnected`` that starts from its
    weight and bias (examples/vitb16_imagenet1k/utils.py:67-77; the ``beta_zero_gain`` argument passed
    there is one the layer does not have, so it is not taken here).  Further keyword arguments go to the
    ``FullyConnected`` constructor (``store_args``, ``compute_exact`` ...)."""
    parents, attributes = get_layers(model, layers_str, True)
    for parent, attr in zip(parents, attributes):
        old = getattr(parent, attr)
        if not isinstance(old, nn.Linear):
            raise TypeError("%s is a %s, not an nn.Linear" % (attr, type(old).__name__))
        has_bias = old.bias is not None
        mam = FullyConnected(old.in_features, old.out_features, bias=has_bias, vcon_steps=vcon_steps,
                             vcon_type=vcon_type, splits=layer_splits, train_mam_only=train_mam_only,
                             device=old.weight.device, dtype=old.weight.dtype, **fc_kwargs)
        mam.weight.data = old.weight.data
        if has_bias:
            mam.bias.data = old.bias.data
        setattr(parent, attr, mam)
    return model


class MAMMlp(nn.Module):
    """The MLP half of a transformer encoder layer with MAM projections: LayerNorm -> FullyConnected
    (hidden -> intermediate) -> GELU -> FullyConnected (intermediate -> hidden), residual added.
    ViT-B/16: hidden 768, intermediate 3072, 197 tokens per image."""

    def __init__(self, hidden: int = 768, intermediate: int = 3072, eps: float = 1e-12, residual: bool = True,
                 device=None, dtype=None, **fc_kwargs):
        super().__init__()
        self.norm = nn.LayerNorm(hidden, eps=eps, device=device, dtype=dtype)
        self.intermediate = FullyConnected(hidden, intermediate, device=device, dtype=dtype, **fc_kwargs)
        self.act = nn.GELU()
        self.output = FullyConnected(intermediate, hidden, device=device, dtype=dtype, **fc_kwargs)
        self.residual = residual

    def vcon_step(self) -> None:
        self.intermediate.vcon_step()
        self.output.vcon_step()

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        y = self.output(self.act(self.intermediate(self.norm(tokens))))
        return tokens + y if self.residual else y
