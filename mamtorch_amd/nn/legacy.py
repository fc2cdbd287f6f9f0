"""The two older MAM layers that the reference still exports, over the same kernels.

``FullyConnectedV1`` mirrors ``mamtorch.nn.v1.FullyConnected`` (mamtorch/nn/v1/fullyconnected.py:8-121):
Xavier-like initialisation chosen by ``init_mode``, a linear vanishing-contribution schedule, and the output
``(1 - beta) * MAM + bias + beta * MAC``.  ``MAMDense`` mirrors the deprecated ``mamtorch.MAMDense``
(mamtorch/nn/compat.py:9-117): Kaiming-uniform initialisation and a per-epoch ``adjust_beta``.

Both always keep ``argmax`` / ``argmin`` of the last call and count selections by the reference's literal
rule (both index sets go into ``max_selection_count``, duplicates within a call count once,
mamtorch/nn/v1/fullyconnected.py:72-86).  Differences from the reference, all deliberate: the weight is used
in its stored (out, in) layout, the bias rides in the kernel when there is no MAC term, the selection count
is one kernel, and a missing argmax raises ``Exception`` (the reference raises a ``str``, a ``TypeError``).
"""
import math

import torch
import torch.nn.functional as F
from torch.nn import Module, Parameter

from .. import kernel as K

__all__ = ["FullyConnectedV1", "MAMDense"]


class _BlendedMAM(Module):
    """Shared part: parameters, selection counting, and the (1 - beta) MAM + beta MAC output."""

    def _uses_mac(self):
        return self.beta > 0

    def _make_parameters(self, in_features, out_features, bias):
        self.weight = Parameter(torch.empty(out_features, in_features))
        if bias:
            self.bias = Parameter(torch.empty(out_features))
        else:
            self.register_parameter("bias", None)
        self.max_selection_count = None
        self.min_selection_count = None
        self.argmax = None
        self.argmin = None

    def reset_selection_count(self):
        shape, dev = self.weight.shape, self.weight.device
        self.max_selection_count = torch.zeros(shape, dtype=torch.int32, device=dev)
        self.min_selection_count = torch.zeros(shape, dtype=torch.int32, device=dev)

    def update_selection_count(self):
        if self.argmax is None or self.argmin is None:
            raise Exception("No argmax or argmin values have been evaluated yet.")
        if self.max_selection_count is None or self.min_selection_count is None:
            self.reset_selection_count()
        K.v4.selection_count(self.argmax, self.argmin, self.max_selection_count, self.min_selection_count,
                             K.v4.COUNT_REFERENCE)

    def forward(self, input):
        rows = input.reshape(-1, input.size(-1))
        blend = self._uses_mac()
        # without a MAC term the bias is added inside the kernel: (max + min) + bias, the reference's order
        fused = self.bias if (self.bias is not None and not blend) else None
        c, self.argmax, self.argmin = K.v4.fullyconnected_wt(rows, self.weight, fused)
        shape = tuple(input.shape[:-1]) + (self.weight.size(0),)
        if not blend:
            return c.view(shape)
        mam = (1 - self.beta) * c
        if self.bias is not None:
            mam = mam + self.bias.view(1, -1)
        return mam.view(shape) + self.beta * F.linear(input, self.weight)


class FullyConnectedV1(_BlendedMAM):

    def __init__(self, in_features, out_features, bias=True, vcon_steps=0, vcon_type='linear', init_mode='uniform',
                 **kwargs):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.use_bias = bias
        self.vcon_type = vcon_type
        self.vcon_steps = vcon_steps
        self.init_mode = init_mode
        self._make_parameters(in_features, out_features, bias)
        self.beta = 1.0 if vcon_steps > 0 else 0.0
        self.reset_parameters()

    def reset_parameters(self):
        # Xavier-like bounds with a fan of 2 + out_features (mamtorch/nn/v1/fullyconnected.py:37-48)
        fan = 2 + self.out_features
        if self.init_mode == "uniform":
            bound = math.sqrt(6 / fan)
            torch.nn.init.uniform_(self.weight, -bound, bound)
        elif self.init_mode == "normal":
            torch.nn.init.normal_(self.weight, std=math.sqrt(2 / fan))
        if self.bias is not None:
            torch.nn.init.zeros_(self.bias)

    def vcon_step(self):
        if self.vcon_steps < 0:
            raise Exception("Invalid value for vcon_steps. Please use 0 or a positive integer.")
        if self.vcon_steps == 0:
            return
        if self.vcon_type != 'linear':
            raise Exception(f"Vanishing contribution type '{self.vcon_type}' is not supported")
        self.beta -= 1 / self.vcon_steps
        if self.beta <= 1e-8:
            self.beta = 0

    def __repr__(self):
        return (f"MAM@FullyConnected(in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.use_bias}, vcon_steps={self.vcon_steps}, vcon_type={self.vcon_type})")


class MAMDense(_BlendedMAM):

    def _uses_mac(self):
        return self.beta >= 10e-5   # mamtorch/nn/compat.py:98

    def __init__(self, in_features, out_features, bias=True, beta=False, beta_decay='linear', beta_epochs=1):
        print("Warning: the use of mamtorch.MAMDense is deprecated. Use mamtorch.nn.FullyConnected instead.")
        super().__init__()
        self.input_features = in_features
        self.state_size = out_features
        self.beta_decay = beta_decay
        self.beta_epochs = beta_epochs
        self._make_parameters(in_features, out_features, bias)
        self.beta = 1.0 if beta else 0.0
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in = self.weight.size(1)
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            torch.nn.init.uniform_(self.bias, -bound, bound)

    def adjust_beta(self, epoch):
        """beta as a function of the epoch (mamtorch/nn/compat.py:45-61); unknown decays leave it alone."""
        if self.beta_epochs < 0:
            raise Exception("Invalid value for beta_epochs. Please use a positive integer.")
        if epoch >= self.beta_epochs:
            self.beta = 0
            return
        t = epoch / self.beta_epochs
        if self.beta_decay == 'linear':
            self.beta = 1 - t
        elif self.beta_decay == 'descending-parabola':
            self.beta = 1 - t ** 2
        elif self.beta_decay == 'ascending-parabola':
            self.beta = 1 + (1 / (self.beta_epochs ** 2) * (epoch ** 2)) - ((2 / self.beta_epochs) * epoch)
