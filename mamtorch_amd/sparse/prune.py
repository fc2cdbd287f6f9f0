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

def _operand(score: Tensor, factor, counts):
    """(w, mode, aux, aux2) for capi.select_abs_ranks: `score` as a 2-d fp32 matrix with contiguous rows."""
    t = score.detach()
    if t.dtype != torch.float32 or t.dim() == 0:
        t = t.float().reshape(1, -1)
    if t.dim() != 2 or t.stride(-1) != 1:
        t = t.reshape(1, -1) if t.is_contiguous() else t.contiguous().reshape(1, -1)
    mode, aux, aux2 = _mode(t, factor, counts)
    if aux is not None:
        aux = aux.reshape(t.shape) if aux.is_contiguous() else aux.contiguous().reshape(t.shape)
    if aux2 is not None:
        aux2 = aux2.reshape(t.shape) if aux2.is_contiguous() else aux2.contiguous().reshape(t.shape)
    return t, mode, aux, aux2


def layer_threshold(score: Tensor, p: float, factor: Tensor = None, counts=None) -> float:
    """``torch.quantile(score.flatten().abs(), p)`` (linear interpolation) without sorting and without
    torch's 16 M element limit: the two neighbours of the quantile are found by a radix select on the device
    (three histogram passes, capi.select_abs_ranks) and interpolated exactly as torch.quantile does it -- the
    rank ``p * (n - 1)`` is formed in fp32, its floor and ceiling are the neighbours, ``lerp`` joins them.
    ``factor`` / ``counts`` choose the score as in :func:`prune_` (weight x factor, selection counts)."""
    operand = _operand(score, factor, counts)
    n = operand[0].numel()
    if n == 0:
        raise ValueError("no scores")
    rank = torch.tensor(p, dtype=torch.float32) * (n - 1)
    lo, hi = int(torch.floor(rank)), int(torch.ceil(rank))
    lo, hi = max(0, min(lo, n - 1)), max(0, min(hi, n - 1))
    found = capi.select_abs_ranks([operand], [lo] if hi == lo else [lo, hi]).cpu()
    below, above = found[0], found[-1]
    return float(torch.lerp(below, above, rank - torch.floor(rank)))


def global_threshold(scores, p: float, factors=None, counts=None) -> float:
    """Element of rank ``int(p * n)`` of the sorted absolute scores of all given tensors, without
    concatenating or sorting them: every histogram pass of the radix select walks the tensors one by one."""
    scores = list(scores)
    factors = [None] * len(scores) if factors is None else list(factors)
    counts = [None] * len(scores) if counts is None else list(counts)
    operands = [_operand(s, f, c) for s, f, c in zip(scores, factors, counts)]
    operands = [o for o in operands if o[0].numel() > 0]
    n = sum(o[0].numel() for o in operands)
    if n == 0:
        raise ValueError("no scores")
    index = max(0, min(int(p * n), n - 1))
    return float(capi.select_abs_ranks(operands, [index]).cpu()[0])


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
