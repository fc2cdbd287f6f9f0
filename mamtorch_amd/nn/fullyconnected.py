"""MAM fully-connected layer: y = max_k(w_jk x_k) + min_k(w_jk x_k) + bias_j.

Drop-in for ``mamtorch.nn.FullyConnected`` (mamtorch/nn/v4/fullyconnected.py:10-221): same
constructor arguments, attributes, exceptions, vanishing-contribution schedule, selection
counting and repr.  What differs is only how the work reaches the GPU:

  * the weight is used in its stored (out, in) layout -- the reference materialises
    ``weight.T.contiguous()`` on every call (:141);
  * the bias add is fused into the kernel when there is no MAC blend and no input split;
  * ``splits > 1`` passes row-strided views to the kernel (the reference hands such views to
    code that assumes contiguous memory, :165-176);
  * every forward kernel is exact, so ``compute_exact`` selects nothing;
  * ``update_selection_count`` is one kernel.  ``selection_count_mode="reference"`` (default)
    keeps the literal behaviour of :123-129 (per call a weight gains 1 if any row picked it as
    max and 1 if any row picked it as min, both added to ``max_selection_count``);
    ``"hits"`` counts every pick and keeps max and min apart.
"""
import math

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.nn import Module, Parameter

from .. import kernel as K

__all__ = ["FullyConnected"]


class FullyConnected(Module):

    __name__ = "FullyConnected"
    __constants__ = ["in_features", "out_features"]
    in_features: int
    out_features: int
    weight: Tensor

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = True,
        splits: int = 1,
        relu_in: bool = False,
        vcon_steps: int = 0,
        vcon_type: str = 'linear',
        vcon_eps: float = 1e-3,
        vcon_expand: bool = False,
        wdrop_rate: float = 0,
        drop_rate: float = 0,
        compute_exact=False,
        train_mam_only=False,
        store_args=False,
        device=None,
        dtype=None,
        selection_count_mode: str = "reference",
    ) -> None:
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()

        self.in_features = in_features
        self.out_features = out_features
        self.splits = splits
        self.relu_in = relu_in
        self.vcon_type = vcon_type
        self.vcon_steps = vcon_steps
        self.vcon_eps = vcon_eps
        self.vcon_expand = vcon_expand
        self.wdrop_rate = wdrop_rate
        self.drop_rate = drop_rate
        self.compute_exact = compute_exact
        self.train_mam_only = train_mam_only
        self.store_args = store_args
        if selection_count_mode not in ("reference", "hits"):
            raise Exception(f"selection_count_mode '{selection_count_mode}' is not supported.")
        self.selection_count_mode = selection_count_mode

        self.weight = Parameter(torch.empty(self.out_features, self.in_features, **factory_kwargs))
        if self.splits > 1:
            self.in_subfeatures = math.ceil(self.in_features / self.splits)
            self.in_subfeatures_last = self.in_features - self.in_subfeatures * (self.splits - 1)

        if bias:
            self.bias = Parameter(torch.empty(out_features, **factory_kwargs))
        else:
            self.register_parameter('bias', None)

        # vanishing contributions: beta weighs the MAC term, alpha the MAM term
        if vcon_steps > 0:
            self.beta = 1.0
            self.alpha = 0.0
        else:
            self.beta = 0.0
            self.alpha = 1.0

        self.max_selection_count = None
        self.min_selection_count = None
        self.argmax = None
        self.argmin = None

        self.reset_parameters()

    def reset_parameters(self) -> None:
        # Kaiming-uniform with a = sqrt(5): U(+-1/sqrt(in_features)) for weight and bias
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = torch.nn.init._calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            torch.nn.init.uniform_(self.bias, -bound, bound)

    def vcon_step(self) -> None:
        if self.vcon_steps < 0:
            raise Exception("Invalid value for vcon_steps. Please use 0 or a positive integer.")
        elif self.vcon_steps == 0:
            return

        if self.vcon_type == 'linear':
            self.beta -= 1 / self.vcon_steps
        elif self.vcon_type == 'exponential':
            self.beta *= math.exp(math.log(self.vcon_eps) / self.vcon_steps)
        else:
            raise Exception(f"vcon_type '{self.vcon_type}' is not supported.")

        if self.beta <= self.vcon_eps:
            self.beta = 0

        self.alpha = 1.0 - self.beta
        if self.vcon_expand:
            self.alpha *= self.in_features / (2 * self.splits)

    def reset_selection_count(self) -> None:
        if not self.store_args:
            raise Exception("MAM layer has not been set to store max and min arguments (store_args is False). Do not use reset_selection_count()")
        self.max_selection_count = torch.zeros(self.weight.shape, dtype=torch.int32, device=self.weight.device)
        self.min_selection_count = torch.zeros(self.weight.shape, dtype=torch.int32, device=self.weight.device)

    def update_selection_count(self) -> None:
        if not self.store_args:
            raise Exception("MAM layer has not been set to store max and min arguments (store_args is False). Do not use update_selection_count()")
        if self.argmax is None or self.argmin is None:
            raise Exception("No argmax or argmin values have been evaluated yet.")
        if self.max_selection_count is None or self.min_selection_count is None:
            self.reset_selection_count()
        mode = K.v4.COUNT_HITS if self.selection_count_mode == "hits" else K.v4.COUNT_REFERENCE
        K.v4.selection_count(self.argmax, self.argmin, self.max_selection_count,
                             self.min_selection_count, mode)

    def _dropped_weight(self) -> Tensor:
        """Weight with the training-time weight dropout applied, still (out, in)."""
        w = self.weight
        if self.training and self.wdrop_rate != 0:
            if not (0 < self.wdrop_rate < 1):
                raise Exception("wdrop_rate must be between 0 and 1.")
            # the reference draws a float mask of the weight's size and multiplies (a second copy of W and
            # three more passes over it); here the mask is one byte per weight, drawn by torch's generator,
            # and one kernel forms weight * mask; autograd masks the weight gradient with the same call
            keep = torch.empty(w.shape, dtype=torch.bool, device=w.device).bernoulli_(1 - self.wdrop_rate)
            w = K.v4.apply_keep(w, keep)
        return w

    def _mam_noargs(self, x: Tensor, w: Tensor, bias) -> Tensor:
        if self.beta < 1:
            if self.training:
                return K.v4.fullyconnected_wt(x, w, bias)[0]
            return K.v4.fullyconnected_fast_wt(x, w, bias)
        return torch.zeros((x.shape[0], w.shape[0]), device=w.device, dtype=w.dtype)

    def forward(self, input: Tensor) -> Tensor:
        if self.relu_in:
            input = F.relu(input)

        input_flat = input.reshape(-1, input.size()[-1])
        w = self._dropped_weight()
        # without a MAC blend the bias rides along in the MAM kernel, after the sum of max and min (and
        # after the sum over the splits): the reference's rounding order; with a blend the blend adds it
        fuse_bias = self.bias is not None and self.beta == 0
        fused = self.bias if fuse_bias and self.splits == 1 else None
        fused_ranges = self.bias if fuse_bias else None

        if self.splits > 1:
            # one operator for all slices: consecutive ranges of in_subfeatures inputs, summed in ascending
            # order and then the bias -- the rounding order of the reference's `C_flat += ...` statements
            if self.beta < 1:
                C_flat = K.v4.fullyconnected_ranges(input_flat, w, fused_ranges, self.in_subfeatures)
            else:
                C_flat = torch.zeros((input_flat.shape[0], w.shape[0]), device=w.device, dtype=w.dtype)
        else:
            if self.store_args:
                C_flat, argmax, argmin = K.v4.fullyconnected_wt(input_flat, w, fused)[:3]
                self.argmax = argmax
                self.argmin = argmin
            else:
                C_flat = self._mam_noargs(input_flat, w, fused)

        if self.beta > 0:
            # alpha * MAM + beta * MAC + bias as one kernel, in the reference's rounding order
            mac_weight = self.weight.detach() if self.train_mam_only else self.weight
            C_flat = K.v4.blend(C_flat, F.linear(input_flat, mac_weight), self.bias, self.alpha, self.beta)

        C = C_flat.view(input.shape[:-1] + (self.weight.size(0),))

        if self.drop_rate > 0:
            C = F.dropout(C, self.drop_rate, self.training)

        return C

    def __repr__(self) -> str:
        s = (f"MAM@FullyConnected(in_features={self.in_features}, out_features={self.out_features}, "
             f"bias={self.bias is not None}")
        if self.vcon_steps > 0:
            s += f", vcon_steps={self.vcon_steps}, vcon_type={self.vcon_type}"
        if self.splits > 1:
            s += f", splits={self.splits}"
        if self.vcon_expand:
            s += ", vcon_expand=True"
        if self.relu_in:
            s += ", relu_in=True"
        return s + ")"
