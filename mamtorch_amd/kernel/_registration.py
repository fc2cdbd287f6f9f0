"""Fake (meta) kernels and autograd formulas shared by the operator namespaces.

Follows mamtorch/kernel/v4/fullyconnected.py:12-64 and mamtorch/kernel/v1/fullyconnected.py:12-64:
the forward saves (a, b) only when a gradient is needed and always saves both index tensors; the
backward calls the namespace's own ``fullyconnected_backward`` with the gradient of C only.
"""
import torch


def _check_forward(a, b):
    torch._check(a.dim() == 2 and b.dim() == 2)
    torch._check(a.size(1) == b.size(0))
    torch._check(a.dtype == torch.float)
    torch._check(b.dtype == torch.float)
    torch._check(a.device == b.device)


def register_exact_forward(ns):
    """ns::fullyconnected(a, b) -> [C, argmax, argmin] and ns::fullyconnected_backward."""
    ops = getattr(torch.ops, ns)

    @torch.library.register_fake(f"{ns}::fullyconnected")
    def _(a, b):
        _check_forward(a, b)
        shape = (a.size(0), b.size(1))
        return [torch.empty(shape, dtype=torch.float, device=a.device),
                torch.empty(shape, dtype=torch.int, device=a.device),
                torch.empty(shape, dtype=torch.int, device=a.device)]

    def _setup_context(ctx, inputs, output):
        a, b = inputs
        _, argmax, argmin = output
        need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        ctx.save_for_backward(a if need else None, b if need else None, argmax, argmin)
        # the index outputs never receive a gradient: without this autograd fills two (N, out) tensors with
        # zeros for them before every backward
        ctx.set_materialize_grads(False)

    def _backward(ctx, grad):
        a, b, argmax, argmin = ctx.saved_tensors
        a_grad, b_grad = None, None
        if grad[0] is not None and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1]):
            a_grad, b_grad = ops.fullyconnected_backward.default(a, b, grad[0].contiguous(), argmax, argmin)
        return a_grad, b_grad

    torch.library.register_autograd(f"{ns}::fullyconnected", _backward, setup_context=_setup_context)

    @torch.library.register_fake(f"{ns}::fullyconnected_backward")
    def _(a, b, grad, argmax, argmin):
        _check_forward(a, b)
        torch._check(grad.size(0) == a.size(0))
        torch._check(grad.size(1) == b.size(1))
        torch._check(grad.shape == argmax.shape)
        torch._check(grad.shape == argmin.shape)
        torch._check(grad.dtype == torch.float)
        torch._check(argmax.dtype == torch.int)
        torch._check(argmin.dtype == torch.int)
        torch._check(argmax.is_contiguous())
        torch._check(argmin.is_contiguous())
        return [torch.empty((a.size(0), a.size(1)), dtype=torch.float, device=a.device),
                torch.empty((b.size(0), b.size(1)), dtype=torch.float, device=a.device)]
