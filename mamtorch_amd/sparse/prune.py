"""Pruning of MAM weights and their compaction to CSR for the sparse kernels.

The rule is the reference's (examples/vitb16_imagenet1k/pruning_utils.py): an entry is removed when
``score.abs() <= threshold``; the score is the weight itself (magnitude pruning, LMP :103-111 / GMP
:152-160), weight x gradient (LGP :190-203 / GGP :252-263) or -- the use the MAM papers make of
``FullyConnected.max_selection_count + min_selection_count`` -- how often the weight was selected.
Thresholds are a quantile of the scores of one layer (``torch.quantile``, :104) or the element of
rank ``int(p * n)`` of the sorted scores of several layers (:139-143).
The reference keeps the pruned matrices dense (``prune_``); ``dense_to_csr`` hands the survivors to
``mamtorch_amd.sparse.fullyconnected`` / ``cusparsemm`` without materialising a mask.
"""
import torch
from torch import Tensor

from .. import capi

__all__ = ["layer_threshold", "global_threshold", "prune_", "dense_to_csr"]

_QUANTILE_LIMIT = 16_000_000  # torch.quantile refuses larger inputs


def layer_threshold(score: Tensor, p: float) -> float:
    """``torch.quantile(score.flatten().abs(), p)`` (linear interpolation), also above torch's size limit."""
    flat = score.detach().flatten().abs().float()
    if flat.numel() <= _QUANTILE_LIMIT:
        return float(torch.quantile(flat, p))
    ordered, _ = torch.sort(flat)
    pos = p * (flat.numel() - 1)
    lo = int(pos)
    hi = min(lo + 1, flat.numel() - 1)
    a, b = ordered[lo], ordered[hi]
    return float(a + (b - a) * (pos - lo))


def global_threshold(scores, p: float) -> float:
    """Element of rank ``int(p * n)`` of the sorted absolute scores of all given tensors."""
    flat = torch.cat([s.detach().flatten().abs().float() for s in scores])
    ordered, _ = torch.sort(flat)
    index = max(0, min(int(p * flat.numel()), flat.numel() - 1))
    return float(ordered[index])


def _mode(weight, factor, counts):
    if factor is not None and counts is not None:
        raise ValueError("give either a factor (weight x factor score) or selection counts, not both")
    if counts is not None:
        a, b = (counts, None) if isinstance(counts, Tensor) else (counts[0], counts[1])
        return capi.PRUNE_COUNT, a.to(torch.int32), None if b is None else b.to(torch.int32)
    if factor is not None:
        return capi.PRUNE_WEIGHT_TIMES, factor.detach().float(), None
    return capi.PRUNE_MAGNITUDE, None, None


def prune_(weight: Tensor, threshold: float, factor: Tensor = None, counts=None) -> Tensor:
    """In place ``weight[score.abs() <= threshold] = 0``.  ``factor``: score = weight * factor (pass the
    gradient); ``counts``: score = the int32 selection counts (a tensor, or a (max, min) pair that is summed)."""
    mode, aux, aux2 = _mode(weight, factor, counts)
    w = weight.detach()
    if w.dim() != 2 or w.dtype != torch.float32 or w.stride(1) != 1:
        raise ValueError("weight must be a 2-d float32 tensor with contiguous rows")
    capi.prune_apply(w, float(threshold), mode, aux, aux2)
    return weight


def dense_to_csr(weight: Tensor, threshold: float = 0.0, factor: Tensor = None, counts=None) -> Tensor:
    """``torch.sparse_csr`` tensor (int64 indices, ascending columns) of the entries that survive the rule
    above.  With the defaults: the non-zero entries, i.e. ``weight.to_sparse_csr()`` of an already pruned
    matrix."""
    mode, aux, aux2 = _mode(weight, factor, counts)
    w = weight.detach()
    if w.dim() != 2 or w.dtype != torch.float32 or w.stride(1) != 1:
        raise ValueError("weight must be a 2-d float32 tensor with contiguous rows")
    crow, col, val = capi.prune_to_csr(w, float(threshold), mode, aux, aux2)
    return torch.sparse_csr_tensor(crow, col, val, size=tuple(w.shape))
