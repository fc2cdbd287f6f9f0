"""MAM convolutions over the MAM fully-connected kernel.

``MAMConv1d`` / ``MAMConv2d`` take the argument lists of the reference's retired modules
(mamtorch/nn/backup/mamconv1d.txt:20-48, mamtorch/nn/backup/mamconv2d.txt:20-58): each output position
is a MAM neuron over its window, ``Y[b, f, l] = max_q p_q + min_q p_q`` with ``p_q`` the products of
the window's inputs and filter ``f``'s weights, and ``argmax`` / ``argmin`` the lowest
``q = position * in_channels + channel`` attaining them (window column outermost in 2-D;
mamtorch/kernel/backup/mamconv1d_forward.txt:128, decoding in mamtorch/nn/backup/mamconv2d.txt:97-103).

The reference ran dedicated kernels on inputs permuted to column-major; here the windows are gathered once
(``kernel.v4.im2col``, a HIP kernel) into a ``(B * L, k * C)`` operand in that index order and the dense MAM
forward / backward do the rest, so the convolutions inherit the exact first-index rule, the hand-over of the
selected operands and the atomics-free backward; the input gradient is the adjoint gather
(``kernel.v4.col2im``).  Outputs are returned in the reference's ``(B, F, L...)`` shape as permuted views.
Messages of the reference's ``raise("...")`` statements (a ``TypeError`` there) are raised as ``Exception``.
"""
import math

import torch
import torch.nn.functional as F
from torch.nn import Module, Parameter

from .. import kernel as K

__all__ = ["MAMConv1d", "MAMConv2d"]


class _MAMConvNd(Module):
    """Shared: parameters, beta schedule, selection counting, and the flat (rows, filters) core."""

    def _init_common(self, in_channels, out_channels, kernel_size, bias, stride, padding, padding_mode, beta,
                     beta_decay, beta_epochs, weight_shape):
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.padding_mode = padding_mode
        self.beta_decay = beta_decay
        self.beta_epochs = beta_epochs
        self.weight = Parameter(torch.empty(weight_shape))
        if bias:
            self.bias = Parameter(torch.empty(out_channels))
        else:
            self.register_parameter("bias", None)
        self.beta = 1.0 if beta else 0.0
        self.max_selection_count = None
        self.min_selection_count = None
        self.argmax = None
        self.argmin = None
        self._flat_args = None
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = torch.nn.init._calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            torch.nn.init.uniform_(self.bias, -bound, bound)

    def adjust_beta(self, epoch):
        if self.beta_epochs <= 0:
            raise Exception("Invalid value for beta_epochs. Please use a positive integer.")
        if epoch >= self.beta_epochs:
            self.beta = 0
            return
        if self.beta_decay == 'linear':
            self.beta = 1 - epoch / self.beta_epochs
        elif self.beta_decay == 'descending-parabola':
            self.beta = 1 - (epoch / self.beta_epochs) ** 2
        elif self.beta_decay == 'ascending-parabola':
            self.beta = 1 + (1 / (self.beta_epochs ** 2) * (epoch ** 2)) - ((2 / self.beta_epochs) * epoch)

    # weight (F, C, k...) <-> the kernel's (F, q) matrix, q = position * C + channel
    def _weight_matrix(self):
        raise NotImplementedError

    def _counts_like_weight(self, flat):
        raise NotImplementedError

    def reset_selection_count(self):
        self.max_selection_count = torch.zeros(self.weight.shape, dtype=torch.int32, device=self.weight.device)
        self.min_selection_count = torch.zeros(self.weight.shape, dtype=torch.int32, device=self.weight.device)

    def update_selection_count(self):
        """The reference's literal rule (mamtorch/nn/backup/mamconv1d.txt:84-103): per call a weight's max
        counter gains 1 if any output position picked it as argmax (an advanced-index ``+= 1`` does not
        accumulate duplicates), its min counter likewise for argmin."""
        if self._flat_args is None:
            raise Exception("No argmax or argmin values have been evaluated yet.")
        if self.max_selection_count is None or self.min_selection_count is None:
            self.reset_selection_count()
        argmax, argmin = self._flat_args
        rows = self.weight.size(0)
        width = self.weight.numel() // rows
        cmax = torch.zeros((rows, width), dtype=torch.int32, device=argmax.device)
        cmin = torch.zeros((rows, width), dtype=torch.int32, device=argmax.device)
        K.v4.selection_count(argmax, argmin, cmax, cmin, K.v4.COUNT_FLAGS)
        self.max_selection_count += self._counts_like_weight(cmax)
        self.min_selection_count += self._counts_like_weight(cmin)

    def _mam(self, X4, k1, k2, s1, s2):
        """X4 (B, C, H, W) padded input -> flat (B * L1 * L2, F) output, and the output positions."""
        B, _, H, W = X4.shape
        L1, L2 = (H - k1) // s1 + 1, (W - k2) // s2 + 1
        cols = K.v4.im2col(X4, k1, k2, s1, s2)
        fused_bias = self.bias if self.beta < 10e-5 else None
        Y, argmax, argmin = K.v4.fullyconnected_wt(cols, self._weight_matrix(), fused_bias)
        self._flat_args = (argmax, argmin)
        return Y, argmax, argmin, (B, L1, L2)

    def _blend(self, Y, Yb_flat):
        # (1 - beta) * Y + beta * Yb + bias, the reference's rounding order
        return K.v4.blend(Y, Yb_flat, self.bias, 1 - self.beta, self.beta)


class MAMConv1d(_MAMConvNd):
    def __init__(self, in_channels, out_channels, kernel_size, bias=True, stride=1, padding=0, padding_mode='zeros',
                 beta=False, beta_decay='linear', beta_epochs=1):
        super().__init__()
        self._init_common(in_channels, out_channels, kernel_size, bias, stride, padding, padding_mode, beta,
                          beta_decay, beta_epochs, (out_channels, in_channels, kernel_size))

    def _weight_matrix(self):
        return self.weight.permute(0, 2, 1).reshape(self.weight.size(0), -1)

    def _counts_like_weight(self, flat):
        Fo, C, k = self.weight.shape
        return flat.view(Fo, k, C).permute(0, 2, 1)

    def _pad(self, input):
        pad_mode = 'constant' if self.padding_mode == 'zeros' else self.padding_mode
        if isinstance(self.padding, (tuple, list)):
            if len(self.padding) <= 2:
                return F.pad(input, tuple(self.padding), mode=pad_mode)
            raise Exception("To much elements in padding list or tuple.")
        if type(self.padding) is int:
            if self.padding == 0:
                return input
            if self.padding > 0:
                padl = self.padding // 2
                return F.pad(input, (padl, self.padding - padl), mode=pad_mode)
            raise Exception("Padding value must be equal or greater than 0.")
        if self.padding == 'same':
            pad_total = self.weight.size(2) - 1
            padl = pad_total // 2
            return F.pad(input, (padl, pad_total - padl), mode=pad_mode)
        if self.padding == 'valid':
            return input
        raise Exception("Invalid padding value.")

    def forward(self, input):
        X = self._pad(input)
        k = self.weight.size(2)
        Y, argmax, argmin, (B, _, L) = self._mam(X.unsqueeze(2), 1, k, 1, self.stride)
        Fo = self.weight.size(0)
        self.argmax = argmax.view(B, L, Fo).permute(0, 2, 1)
        self.argmin = argmin.view(B, L, Fo).permute(0, 2, 1)
        if self.beta >= 10e-5:
            Yb = F.conv1d(X, self.weight, stride=self.stride)
            Y = self._blend(Y, Yb.permute(0, 2, 1).reshape(B * L, Fo))
        return Y.view(B, L, Fo).permute(0, 2, 1)


class MAMConv2d(_MAMConvNd):
    def __init__(self, in_channels, out_channels, kernel_size, bias=True, stride=1, padding=0, padding_mode='zeros',
                 beta=False, beta_decay='linear', beta_epochs=1):
        super().__init__()
        if isinstance(kernel_size, (tuple, list)):
            shape = (out_channels, in_channels, kernel_size[0], kernel_size[1])
        else:
            shape = (out_channels, in_channels, kernel_size, kernel_size)
        if type(stride) is tuple:
            self.hstride, self.wstride = stride
        else:
            self.hstride = self.wstride = stride
        self._init_common(in_channels, out_channels, kernel_size, bias, stride, padding, padding_mode, beta,
                          beta_decay, beta_epochs, shape)

    def _weight_matrix(self):
        # q = (window column * window rows + window row) * C + channel
        return self.weight.permute(0, 3, 2, 1).reshape(self.weight.size(0), -1)

    def _counts_like_weight(self, flat):
        Fo, C, k1, k2 = self.weight.shape
        return flat.view(Fo, k2, k1, C).permute(0, 3, 2, 1)

    def _pad(self, input):
        pad_mode = 'constant' if self.padding_mode == 'zeros' else self.padding_mode
        if isinstance(self.padding, (tuple, list)):
            if len(self.padding) <= 2:
                return F.pad(input, tuple(self.padding), mode=pad_mode)
            if len(self.padding) <= 4:
                return F.pad(input, tuple(self.padding), mode=pad_mode)
            raise Exception("To much elements in padding list or tuple.")
        if type(self.padding) is int:
            if self.padding == 0:
                return input
            if self.padding > 0:
                padl = self.padding // 2
                padr = self.padding - padl
                return F.pad(input, (padl, padr, padl, padr), mode=pad_mode)
            raise Exception("Padding value must be equal or greater than 0.")
        if self.padding == 'same':
            if self.hstride != 1 or self.wstride != 1:
                raise Exception("Cannot apply 'same' padding with stride > 1.")
            pad_w, pad_h = self.weight.size(3) - 1, self.weight.size(2) - 1
            return F.pad(input, (pad_w // 2, pad_w - pad_w // 2, pad_h // 2, pad_h - pad_h // 2), mode=pad_mode)
        if self.padding == 'valid':
            return input
        raise Exception("Invalid padding value.")

    def forward(self, input):
        X = self._pad(input)
        k1, k2 = self.weight.size(2), self.weight.size(3)
        Y, argmax, argmin, (B, L1, L2) = self._mam(X, k1, k2, self.hstride, self.wstride)
        Fo = self.weight.size(0)
        self.argmax = argmax.view(B, L1, L2, Fo).permute(0, 3, 1, 2)
        self.argmin = argmin.view(B, L1, L2, Fo).permute(0, 3, 1, 2)
        if self.beta >= 10e-5:
            Yb = F.conv2d(X, self.weight, stride=(self.hstride, self.wstride))
            Y = self._blend(Y, Yb.permute(0, 2, 3, 1).reshape(B * L1 * L2, Fo))
        return Y.view(B, L1, L2, Fo).permute(0, 3, 1, 2)
