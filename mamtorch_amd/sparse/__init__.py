"""Sparse operators over pruned weights.

``kernel.v1.cusparsemm`` is the reference's sum-of-products SpMM under its own name
(mamtorch/sparse/kernel/v1/cusparsemm.py:9-10).  The CSR-sparse MAM operators, which the reference
does not have, keep that operator's CSR operand convention (int64 crow/col, fp32 values, sparse
operand dispatched on the sparse-CSR key).
"""
from . import kernel
from . import prune
from .fullyconnected import (fullyconnected, fullyconnected_backward, SparseFullyConnectedFunction, prune_to_csr,
                             validate_csr)

__all__ = ["kernel", "prune", "fullyconnected", "fullyconnected_backward", "SparseFullyConnectedFunction", "prune_to_csr",
           "validate_csr"]
