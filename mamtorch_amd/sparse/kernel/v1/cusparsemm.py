"""``mamtorch_kernel_sparsev1::cusparsemm``: sparse (COO or CSR) @ dense -> dense, fp32.

Same name, schema, dispatch keys and fake kernel as mamtorch/sparse/kernel/v1/cusparsemm.py:6-18
and mamtorch/sparse/kernel/v1/csrc/cuda/register_functions.cu:18-28; the implementation behind it
is a hand-written HIP SpMM instead of cuSPARSE.
"""
import torch
from torch import Tensor

__all__ = ["cusparsemm"]

library_name = "mamtorch_kernel_sparsev1"
K = torch.ops.mamtorch_kernel_sparsev1


def cusparsemm(a: Tensor, b: Tensor) -> Tensor:
    """a (rows, k) torch.sparse_coo or torch.sparse_csr, b (k, cols) dense -> (rows, cols) dense."""
    return K.cusparsemm.default(a, b)


@torch.library.register_fake(f"{library_name}::cusparsemm")
def _(a, b):
    torch._check(a.size(1) == b.size(0))
    torch._check(a.dtype == torch.float)
    torch._check(b.dtype == torch.float)
    torch._check(a.device == b.device)
    return torch.empty((a.size(0), b.size(1)), dtype=torch.float, device=a.device)
