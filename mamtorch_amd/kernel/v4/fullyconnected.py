"""``mamtorch_kernel_v4::fullyconnected`` wrapper (mamtorch/kernel/v4/fullyconnected.py:6-64).

The reference's v4 kernel is approximate (index packed into the low mantissa bits,
mamtorch/kernel/v4/csrc/cuda/fullyconnected_kernel.cu:133-137); here the same operator name is
served by the exact kernel, so its error against the oracle is zero.

``fullyconnected_wt`` is an addition: it takes the module's ``weight`` (out, in) as stored, so no
transposed copy of the weight is made per call, adds the bias inside the kernel, and returns the
weight gradient in (out, in) layout.  With ``hand_over`` the raw operator returns a fourth tensor of
shape (4, N, out): the selected weights w[argmax], w[argmin] and the selected inputs x[argmax],
x[argmin].  The index resolution has them in hand, and the backward then needs no random reads of
the weight matrix or of the input.
"""
import torch
from torch import Tensor

from .._registration import register_exact_forward

__all__ = ["fullyconnected", "fullyconnected_wt"]

library_name = "mamtorch_kernel_v4"
K = torch.ops.mamtorch_kernel_v4


def fullyconnected(a: Tensor, b: Tensor) -> list[Tensor]:
    return K.fullyconnected.default(a, b)


def fullyconnected_wt(a: Tensor, weight: Tensor, bias=None) -> list[Tensor]:
    """a (N, in), weight (out, in), bias (out) or None -> [C, argmax, argmin]."""
    # the selected operands are only worth writing when a backward will read them
    hand_over = torch.is_grad_enabled() and (a.requires_grad or weight.requires_grad)
    return K.fullyconnected_wt.default(a, weight, bias, hand_over)[:3]


register_exact_forward(library_name)


@torch.library.register_fake(f"{library_name}::fullyconnected_wt")
def _(a, weight, bias, hand_over):
    torch._check(a.dim() == 2 and weight.dim() == 2)
    torch._check(a.size(1) == weight.size(1))
    torch._check(a.dtype == torch.float)
    torch._check(weight.dtype == torch.float)
    torch._check(a.device == weight.device)
    shape = (a.size(0), weight.size(0))
    return [torch.empty(shape, dtype=torch.float, device=a.device),
            torch.empty(shape, dtype=torch.int, device=a.device),
            torch.empty(shape, dtype=torch.int, device=a.device),
            torch.empty((4 if hand_over else 0,) + shape, dtype=torch.float, device=a.device)]


@torch.library.register_fake(f"{library_name}::fullyconnected_wt_backward")
def _(a, weight, grad, argmax, argmin, sel):
    torch._check(a.size(1) == weight.size(1))
    torch._check(grad.size(0) == a.size(0))
    torch._check(grad.size(1) == weight.size(0))
    torch._check(grad.shape == argmax.shape)
    torch._check(grad.shape == argmin.shape)
    torch._check(argmax.dtype == torch.int)
    torch._check(argmin.dtype == torch.int)
    return [torch.empty((a.size(0), a.size(1)), dtype=torch.float, device=a.device),
            torch.empty((weight.size(0), weight.size(1)), dtype=torch.float, device=a.device)]


def _wt_setup_context(ctx, inputs, output):
    a, weight, bias = inputs[:3]
    _, argmax, argmin, sel = output
    need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
    ctx.save_for_backward(a if need else None, weight if need else None, argmax, argmin,
                          sel if need else None)
    # argmax, argmin and the hand-over tensor never receive a gradient: without this autograd fills three
    # tensors (2 x (N, out) int32 and (4, N, out) fp32) with zeros before every backward
    ctx.set_materialize_grads(False)


def _wt_backward(ctx, grad):
    a, weight, argmax, argmin, sel = ctx.saved_tensors
    a_grad, w_grad, bias_grad = None, None, None
    g = grad[0]
    if g is None:
        return None, None, None, None
    if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
        a_grad, w_grad = K.fullyconnected_wt_backward.default(a, weight, g.contiguous(), argmax, argmin, sel)
    if ctx.needs_input_grad[2]:
        bias_grad = K.bias_grad.default(g)
    return a_grad, w_grad, bias_grad, None


torch.library.register_autograd(
    f"{library_name}::fullyconnected_wt", _wt_backward, setup_context=_wt_setup_context)
