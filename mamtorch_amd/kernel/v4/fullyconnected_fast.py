"""``mamtorch_kernel_v4::fullyconnected_fast`` wrapper (mamtorch/kernel/v4/fullyconnected_fast.py:6-39).

Values only, exact.  As in the reference, its registered backward is the dense multiply-accumulate
gradient (grad @ b.T, a.T @ grad; mamtorch/kernel/v4/fullyconnected_fast.py:22-28), not the MAM
gradient: the module uses this operator in eval mode only.
"""
import torch
from torch import Tensor

__all__ = ["fullyconnected_fast", "fullyconnected_fast_wt"]

library_name = "mamtorch_kernel_v4"
K = torch.ops.mamtorch_kernel_v4


def fullyconnected_fast(a: Tensor, b: Tensor) -> Tensor:
    return K.fullyconnected_fast.default(a, b)


def fullyconnected_fast_wt(a: Tensor, weight: Tensor, bias=None) -> Tensor:
    """Same with ``weight`` in (out, in) layout and the bias added in the kernel."""
    return K.fullyconnected_fast_wt.default(a, weight, bias)


@torch.library.register_fake(f"{library_name}::fullyconnected_fast")
def _(a, b):
    torch._check(a.dim() == 2 and b.dim() == 2)
    torch._check(a.size(1) == b.size(0))
    torch._check(a.dtype == torch.float)
    torch._check(b.dtype == torch.float)
    torch._check(a.device == b.device)
    return torch.empty((a.size(0), b.size(1)), dtype=torch.float, device=a.device)


def _setup_context(ctx, inputs, output):
    a, b = inputs
    need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
    ctx.save_for_backward(a if need else None, b if need else None)


def _backward(ctx, grad):
    a, b = ctx.saved_tensors
    a_grad, b_grad = None, None
    if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
        a_grad = grad @ b.T
        b_grad = a.T @ grad
    return a_grad, b_grad


torch.library.register_autograd(
    f"{library_name}::fullyconnected_fast", _backward, setup_context=_setup_context)


@torch.library.register_fake(f"{library_name}::fullyconnected_fast_wt")
def _(a, weight, bias):
    torch._check(a.dim() == 2 and weight.dim() == 2)
    torch._check(a.size(1) == weight.size(1))
    torch._check(a.dtype == torch.float)
    torch._check(weight.dtype == torch.float)
    return torch.empty((a.size(0), weight.size(0)), dtype=torch.float, device=a.device)


def _wt_setup_context(ctx, inputs, output):
    a, weight, bias = inputs
    need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
    ctx.save_for_backward(a if need else None, weight if need else None)


def _wt_backward(ctx, grad):
    a, weight = ctx.saved_tensors
    a_grad, w_grad, bias_grad = None, None, None
    if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
        a_grad = grad @ weight
        w_grad = grad.T @ a
    if ctx.needs_input_grad[2]:
        bias_grad = grad.sum(dim=0)
    return a_grad, w_grad, bias_grad


torch.library.register_autograd(
    f"{library_name}::fullyconnected_fast_wt", _wt_backward, setup_context=_wt_setup_context)
