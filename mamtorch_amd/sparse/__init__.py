"""CSR-sparse MAM over pruned weights.

The reference's ``mamtorch.sparse`` holds only a cuSPARSE sum-of-products SpMM
(mamtorch/sparse/kernel/v1/cusparsemm.py:9-10); its CSR operand convention (int64 crow/col,
fp32 values, sparse operand first in the reference's SpMM, dispatched on the sparse-CSR key) is
kept for the MAM operators defined here.
"""
from .fullyconnected import fullyconnected, fullyconnected_backward, SparseFullyConnectedFunction, prune_to_csr

__all__ = ["fullyconnected", "fullyconnected_backward", "SparseFullyConnectedFunction", "prune_to_csr"]
