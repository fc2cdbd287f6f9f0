"""Selection-count accumulation as one HIP kernel (no upstream operator name).

Stands in for the two advanced-index updates of FullyConnected.update_selection_count
(mamtorch/nn/v4/fullyconnected.py:123-129).
"""
import torch
from torch import Tensor

__all__ = ["selection_count", "COUNT_REFERENCE", "COUNT_HITS", "COUNT_FLAGS"]

COUNT_REFERENCE = 0  # literal module behaviour: de-duplicated per call, both into max_count
COUNT_HITS = 1       # true hit counts, argmax into max_count and argmin into min_count
COUNT_FLAGS = 2      # de-duplicated per call like COUNT_REFERENCE, but max and min into their own counters

K = torch.ops.mamtorch_kernel_v4


def selection_count(argmax: Tensor, argmin: Tensor, max_count: Tensor, min_count: Tensor,
                    mode: int = COUNT_REFERENCE) -> None:
    """Adds this batch's picks into the (out, in) int32 counters in place."""
    K.selection_count.default(argmax, argmin, max_count, min_count, mode)


@torch.library.register_fake("mamtorch_kernel_v4::selection_count")
def _(argmax, argmin, max_count, min_count, mode):
    torch._check(argmax.shape == argmin.shape)
    torch._check(max_count.shape == min_count.shape)
    torch._check(argmax.size(1) == max_count.size(0))
    return None
