"""``mamtorch_kernel_v1::fullyconnected`` wrapper (mamtorch/kernel/v1/fullyconnected.py:6-10)."""
import torch
from torch import Tensor

from .._registration import register_exact_forward

__all__ = ["fullyconnected"]

library_name = "mamtorch_kernel_v1"
K = torch.ops.mamtorch_kernel_v1


def fullyconnected(a: Tensor, b: Tensor) -> list[Tensor]:
    """a (N, in), b (in, out) -> [C (N, out), argmax int32, argmin int32]; exact, lowest index on ties."""
    return K.fullyconnected.default(a, b)


register_exact_forward(library_name)
