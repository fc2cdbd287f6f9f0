"""``mamtorch_kernel_sparsev1::fullyconnected`` / ``fullyconnected_backward`` wrappers.

``w_csr`` is the pruned weight (out_features, in_features) as a ``torch.sparse_csr`` tensor with
ascending column indices per row (what ``Tensor.to_sparse_csr()`` produces).  The forward result
equals the dense MAM forward on ``w_csr.to_dense()``: entries that were pruned away are zero
weights whose products x*0 take part in the max / min and in the first-index tie-break.
"""
import torch
from torch import Tensor

__all__ = ["fullyconnected", "fullyconnected_backward", "SparseFullyConnectedFunction", "prune_to_csr",
           "validate_csr"]

K = torch.ops.mamtorch_kernel_sparsev1


def fullyconnected(a: Tensor, w_csr: Tensor) -> list[Tensor]:
    """a (N, in) dense, w_csr (out, in) CSR -> [C (N, out), argmax int32, argmin int32]."""
    return K.fullyconnected.default(a, w_csr)


def fullyconnected_backward(a: Tensor, w_csr: Tensor, grad: Tensor, argmax: Tensor, argmin: Tensor) -> list[Tensor]:
    """-> [a_grad (N, in) dense, values_grad (nnz)]; pruned positions receive no gradient."""
    return K.fullyconnected_backward.default(a, w_csr, grad, argmax, argmin)


class SparseFullyConnectedFunction(torch.autograd.Function):
    """Differentiable CSR MAM: gradients flow to ``a`` and to the stored ``values``."""

    @staticmethod
    def forward(ctx, a, values, crow_indices, col_indices, out_features):
        w_csr = torch.sparse_csr_tensor(crow_indices, col_indices, values.detach(),
                                        size=(out_features, a.size(1)))
        # the forward hands the selected values and their positions in `values` to the backward
        c, argmax, argmin, w_sel, pos_sel = K.fullyconnected_sel.default(a.detach(), w_csr)
        ctx.save_for_backward(a, values, crow_indices, col_indices, argmax, argmin, w_sel, pos_sel)
        ctx.out_features = out_features
        ctx.mark_non_differentiable(argmax, argmin)
        return c, argmax, argmin

    @staticmethod
    def backward(ctx, grad, _gmax, _gmin):
        a, values, crow_indices, col_indices, argmax, argmin, w_sel, pos_sel = ctx.saved_tensors
        w_csr = torch.sparse_csr_tensor(crow_indices, col_indices, values.detach(),
                                        size=(ctx.out_features, a.size(1)))
        a_grad, v_grad = K.fullyconnected_sel_backward.default(a.detach(), w_csr, grad.contiguous(), argmax, argmin,
                                                               w_sel, pos_sel)
        return a_grad, v_grad, None, None, None


def prune_to_csr(weight: Tensor, keep_mask: Tensor) -> Tensor:
    """CSR tensor holding ``weight`` where ``keep_mask`` is true (kept zeros stay stored)."""
    mask = keep_mask.to(torch.bool)
    counts = mask.sum(dim=1)
    crow = torch.zeros(weight.size(0) + 1, dtype=torch.int64, device=weight.device)
    crow[1:] = torch.cumsum(counts, dim=0)
    col = mask.nonzero()[:, 1].to(torch.int64)
    return torch.sparse_csr_tensor(crow, col, weight[mask], size=tuple(weight.shape))


def validate_csr(w_csr: Tensor) -> None:
    """Raises ``ValueError`` unless ``w_csr`` satisfies what the sparse kernels take for granted: row offsets
    from 0 to nnz and non-decreasing, column indices inside [0, in_features) and strictly ascending within
    a row.  The operators themselves do not check (a check needs a device round trip per call, and
    ``torch.sparse_csr_tensor`` builds unchecked tensors by default), so call this once on a tensor that
    did not come from ``Tensor.to_sparse_csr()`` / ``sparse.prune`` before handing it to them: a malformed
    tensor makes the kernels read out of range, and the COO SpMM write out of range (its result rows come
    from the row indices).  The dense route of ``cusparsemm`` (``mam_csr_to_dense`` / ``mam_coo_to_dense``)
    writes too, and for that reason drops every entry whose coordinates lie outside the matrix."""
    from .. import capi

    if w_csr.layout != torch.sparse_csr or w_csr.dim() != 2:
        raise ValueError("w_csr must be a 2-dimensional torch.sparse_csr tensor")
    crow = w_csr.crow_indices().to(torch.int64).contiguous()
    col = w_csr.col_indices().to(torch.int64).contiguous()
    if crow.numel() != w_csr.size(0) + 1 or col.numel() != w_csr.values().numel():
        raise ValueError("w_csr: crow_indices / col_indices / values have inconsistent lengths")
    bad = capi.csr_validate(crow, col, w_csr.size(1))
    if bad:
        what = [text for bit, text in ((1, "row offsets do not run from 0 to nnz"), (2, "row offsets decrease"),
                                       (4, "a column index is out of range"),
                                       (8, "column indices are not strictly ascending within a row")) if bad & bit]
        raise ValueError("w_csr is malformed: " + "; ".join(what))
