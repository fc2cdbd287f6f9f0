"""Operators behind the module-level extras (no upstream operator names): the vanishing-contribution
blend of ``FullyConnected`` (mamtorch/nn/v4/fullyconnected.py:190-198) as one kernel, and the window
gather / scatter that feeds the MAM fully-connected kernel with convolution windows
(mamtorch/kernel/backup/mamconv1d_forward.txt, mamconv2d_forward.txt)."""
import torch
from torch import Tensor

__all__ = ["blend", "apply_keep", "im2col", "col2im", "fullyconnected_ranges"]

K = torch.ops.mamtorch_kernel_v4


def fullyconnected_ranges(a: Tensor, weight: Tensor, bias, range_len: int) -> Tensor:
    """The module's `splits` as one operator: the inputs are cut into consecutive ranges of ``range_len``
    (the last one shorter), every range is a MAM neuron of its own, and the result is the sum of the ranges'
    max + min in ascending range order, then the bias.  a (N, in), weight (out, in) -> C (N, out).
    Indices are only computed when a gradient will need them."""
    with_indices = torch.is_grad_enabled() and (a.requires_grad or weight.requires_grad)
    return K.fullyconnected_ranges.default(a, weight, bias, range_len, with_indices)[0]


@torch.library.register_fake("mamtorch_kernel_v4::fullyconnected_ranges")
def _(a, weight, bias, range_len, with_indices):
    torch._check(a.dim() == 2 and weight.dim() == 2 and a.size(1) == weight.size(1))
    torch._check(a.dtype == torch.float and weight.dtype == torch.float)
    ranges = max(1, -(-a.size(1) // range_len)) if with_indices else 0
    shape = (a.size(0), weight.size(0))
    return [torch.empty(shape, dtype=torch.float, device=a.device),
            torch.empty((ranges,) + shape, dtype=torch.int, device=a.device),
            torch.empty((ranges,) + shape, dtype=torch.int, device=a.device)]


@torch.library.register_fake("mamtorch_kernel_v4::fullyconnected_ranges_backward")
def _(a, weight, grad, argmax, argmin, range_len):
    torch._check(a.size(1) == weight.size(1) and grad.size(0) == a.size(0) and grad.size(1) == weight.size(0))
    return [torch.empty(a.shape, dtype=torch.float, device=a.device),
            torch.empty(weight.shape, dtype=torch.float, device=a.device)]


def _ranges_setup(ctx, inputs, output):
    a, weight, _, range_len, with_indices = inputs
    _, argmax, argmin = output
    need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
    ctx.range_len, ctx.with_indices = range_len, with_indices
    ctx.save_for_backward(a if need else None, weight if need else None, argmax, argmin)
    ctx.set_materialize_grads(False)      # no zero-filled gradients for the index outputs


def _ranges_backward(ctx, grad):
    a, weight, argmax, argmin = ctx.saved_tensors
    a_grad = w_grad = bias_grad = None
    g = grad[0]
    if g is None:
        return None, None, None, None, None
    if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
        if not ctx.with_indices:
            raise RuntimeError("fullyconnected_ranges was run without indices; its gradient needs them")
        a_grad, w_grad = K.fullyconnected_ranges_backward.default(a, weight, g.contiguous(), argmax, argmin,
                                                                  ctx.range_len)
    if ctx.needs_input_grad[2]:
        bias_grad = K.bias_grad.default(g)
    return a_grad, w_grad, bias_grad, None, None


torch.library.register_autograd("mamtorch_kernel_v4::fullyconnected_ranges", _ranges_backward,
                                setup_context=_ranges_setup)


def blend(mam: Tensor, mac: Tensor, bias, alpha: float, beta: float) -> Tensor:
    """(alpha * mam + beta * mac) + bias in the reference's rounding order; (N, out) operands."""
    return K.blend.default(mam, mac, bias, float(alpha), float(beta))


def apply_keep(weight: Tensor, keep: Tensor) -> Tensor:
    """weight (out, in) * keep, keep a bool / uint8 mask of the same shape: the weight dropout of
    ``FullyConnected`` (mamtorch/nn/v4/fullyconnected.py:143-148) in one pass; its gradient is the same
    masking of the incoming gradient."""
    return K.apply_keep.default(weight, keep)


def im2col(x: Tensor, k1: int, k2: int, s1: int, s2: int) -> Tensor:
    """x (B, C, H, W) -> (B * L1 * L2, k2 * k1 * C) windows, column (j2 * k1 + j1) * C + c."""
    return K.im2col.default(x, k1, k2, s1, s2)


def col2im(cols: Tensor, shape, k1: int, k2: int, s1: int, s2: int) -> Tensor:
    """Adjoint of :func:`im2col`: (B * L1 * L2, k2 * k1 * C) -> (B, C, H, W), overlapping windows add up."""
    B, C, H, W = shape
    return K.col2im.default(cols, B, C, H, W, k1, k2, s1, s2)


@torch.library.register_fake("mamtorch_kernel_v4::bias_grad")
def _(grad):
    torch._check(grad.dim() == 2 and grad.dtype == torch.float)
    return torch.empty((grad.size(1),), dtype=torch.float, device=grad.device)


@torch.library.register_fake("mamtorch_kernel_v4::blend")
def _(mam, mac, bias, alpha, beta):
    torch._check(mam.dim() == 2 and mam.shape == mac.shape)
    torch._check(mam.dtype == torch.float and mac.dtype == torch.float)
    return torch.empty(mam.shape, dtype=torch.float, device=mam.device)


def _blend_setup(ctx, inputs, output):
    _, _, _, alpha, beta = inputs
    ctx.alpha, ctx.beta = alpha, beta


def _blend_backward(ctx, grad):
    g_mam = grad * ctx.alpha if ctx.needs_input_grad[0] else None
    g_mac = grad * ctx.beta if ctx.needs_input_grad[1] else None
    g_bias = grad.sum(dim=0) if ctx.needs_input_grad[2] else None
    return g_mam, g_mac, g_bias, None, None


torch.library.register_autograd("mamtorch_kernel_v4::blend", _blend_backward, setup_context=_blend_setup)


@torch.library.register_fake("mamtorch_kernel_v4::apply_keep")
def _(weight, keep):
    torch._check(weight.dim() == 2 and weight.dtype == torch.float and keep.shape == weight.shape)
    return torch.empty(weight.shape, dtype=torch.float, device=weight.device)


def _keep_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[1])


def _keep_backward(ctx, grad):
    (keep,) = ctx.saved_tensors
    return K.apply_keep.default(grad, keep), None


torch.library.register_autograd("mamtorch_kernel_v4::apply_keep", _keep_backward, setup_context=_keep_setup)


def _out_positions(H, W, k1, k2, s1, s2):
    return (H - k1) // s1 + 1, (W - k2) // s2 + 1


@torch.library.register_fake("mamtorch_kernel_v4::im2col")
def _(x, k1, k2, s1, s2):
    torch._check(x.dim() == 4 and x.dtype == torch.float)
    B, C, H, W = x.shape
    L1, L2 = _out_positions(H, W, k1, k2, s1, s2)
    return torch.empty((B * L1 * L2, k2 * k1 * C), dtype=torch.float, device=x.device)


@torch.library.register_fake("mamtorch_kernel_v4::col2im")
def _(cols, B, C, H, W, k1, k2, s1, s2):
    torch._check(cols.dim() == 2 and cols.dtype == torch.float)
    return torch.empty((B, C, H, W), dtype=torch.float, device=cols.device)


def _im2col_setup(ctx, inputs, output):
    x, k1, k2, s1, s2 = inputs
    ctx.geom = (tuple(x.shape), k1, k2, s1, s2)


def _im2col_backward(ctx, grad):
    shape, k1, k2, s1, s2 = ctx.geom
    return K.col2im.default(grad.contiguous(), *shape, k1, k2, s1, s2), None, None, None, None


torch.library.register_autograd("mamtorch_kernel_v4::im2col", _im2col_backward, setup_context=_im2col_setup)


def _col2im_setup(ctx, inputs, output):
    ctx.geom = inputs[5:]


def _col2im_backward(ctx, grad):
    k1, k2, s1, s2 = ctx.geom
    return (K.im2col.default(grad.contiguous(), k1, k2, s1, s2),) + (None,) * 8


torch.library.register_autograd("mamtorch_kernel_v4::col2im", _col2im_backward, setup_context=_col2im_setup)
