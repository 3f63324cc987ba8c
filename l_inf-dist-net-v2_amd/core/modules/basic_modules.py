"""Interval-aware building blocks around the distance layers (drop-in for the reference's
core/modules/basic_modules.py).  Every layer maps a triple (x, lower, upper) of optional tensors to a triple; the
element-wise and GEMM work here is plain torch (rocBLAS / MIOpen underneath), there is no hand-written kernel.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F


def apply_if_not_none(paras, func):
    """Map `func` over the entries that are tensors, keep the None placeholders."""
    return [func(t) if t is not None else None for t in paras]


class BoundSequential(nn.Sequential):
    """Sequential over layers that take and return the (x, lower, upper) triple (reference: basic_modules.py:138-142)."""

    def forward(self, paras):
        for layer in self:
            paras = layer(*paras)
        return paras


class MeanShift(nn.Module):
    """Subtracts the per-channel mean: the batch mean (differentiable) in training, with an exponential moving
    average kept in `running_mean` for evaluation (reference: basic_modules.py:104-135).
    Inputs are [B, C, H*W]."""

    def __init__(self, out_channels, momentum=0.1, affine=True):
        super().__init__()
        self.out_channels, self.momentum, self.affine = out_channels, momentum, affine
        self.register_buffer('running_mean', torch.zeros(out_channels))
        self.register_parameter('bias', nn.Parameter(torch.zeros(out_channels)) if affine else None)
        MeanShift.tag = getattr(MeanShift, 'tag', 0) + 1
        self.tag = MeanShift.tag

    def forward(self, x=None, lower=None, upper=None):
        lead = next((t for t in (x, lower, upper) if t is not None), None)
        if lead is not None and lead.is_cuda and lead.dtype == torch.float32 and lead.dim() == 3:
            from core.norm_dist import mean_shift_bias  # the same arithmetic in one fused call of the library
            return mean_shift_bias(x, lower, upper, self.running_mean, self.momentum, self.training, self.bias)
        if self.training:
            assert x is not None, 'Currently not supported'
            mean = x.mean(dim=[0, 2])
            with torch.no_grad():
                self.running_mean.mul_(1 - self.momentum).add_(mean, alpha=self.momentum)
        else:
            mean = self.running_mean
        if self.bias is not None:
            mean = mean - self.bias
        shift = mean.unsqueeze(-1)
        return apply_if_not_none((x, lower, upper), lambda t: t - shift)

    def extra_repr(self):
        return '%d, affine=%s' % (self.out_channels, self.affine)


def linear(input, weight, bias, w_scale, b_scale):
    """w_scale * input @ weight.T + b_scale * bias (reference: basic_modules.py:22-25)."""
    product = input @ weight.t()
    if bias is None:
        return product * w_scale
    return torch.add(bias * b_scale, product, alpha=w_scale)


def _center_radius(lower, upper):
    # twice the centre and twice the radius of the box: the halving is folded into the weight scale
    return lower + upper, upper - lower


def _scaled_init(layer, fan_in, w_scale, b_scale):
    """N(0,1) weights whose 1 / sqrt(fan_in) lives in the forward's scale, zero bias."""
    nn.init.normal_(layer.weight)
    if layer.bias is not None:
        nn.init.zeros_(layer.bias)
    layer.w_scale, layer.b_scale = w_scale / math.sqrt(fan_in), b_scale


class BoundFinalLinear(nn.Linear):
    """Last linear layer: besides the logits it returns, for every sample, the upper bound of
    (logit_j - logit_target) over the input box (reference: basic_modules.py:81-101)."""

    def __init__(self, in_features, out_features, bias=True, w_scale=1.0, b_scale=1.0):
        super().__init__(in_features, out_features, bias=bias)
        _scaled_init(self, in_features, w_scale, b_scale)

    def forward(self, x=None, lower=None, upper=None, targets=None):
        have_box = lower is not None and upper is not None and targets is not None
        if x is not None:
            x = linear(x, self.weight, self.bias, self.w_scale, self.b_scale)
            if not have_box:
                return x
        res = None
        if have_box:
            # per-sample difference rows  W_j - W_target : [B, CO, CI]
            dw = self.weight - self.weight.index_select(0, targets).unsqueeze(1)
            c2, r2 = _center_radius(lower, upper)
            mid = dw.bmm(c2.unsqueeze(-1)) * (self.w_scale / 2)
            if self.bias is not None:
                db = self.bias - self.bias.index_select(0, targets).unsqueeze(1)
                mid = mid + db.unsqueeze(-1) * self.b_scale
            spread = dw.abs().bmm(r2.unsqueeze(-1)) * (self.w_scale / 2)
            res = (mid + spread).squeeze(-1)
        return x, res


class BoundLinear(nn.Linear):
    """Linear layer with N(0,1) weights scaled by w_scale / sqrt(fan_in); interval propagation by
    centre / radius arithmetic W c +- |W| r (reference: basic_modules.py:28-49)."""

    def __init__(self, in_features, out_features, bias=True, w_scale=1.0, b_scale=1.0):
        super().__init__(in_features, out_features, bias=bias)
        _scaled_init(self, in_features, w_scale, b_scale)

    def forward(self, x=None, lower=None, upper=None):
        if x is not None:
            x = linear(x, self.weight, self.bias, self.w_scale, self.b_scale)
        if lower is not None and upper is not None:
            c2, r2 = _center_radius(lower, upper)
            mid = linear(c2, self.weight, self.bias, self.w_scale / 2, self.b_scale)
            spread = (r2 @ self.weight.abs().t()) * (self.w_scale / 2)
            lower, upper = mid - spread, mid + spread
        return x, lower, upper


class BoundConv2d(nn.Conv2d):
    """Convolution counterpart of BoundLinear (reference: basic_modules.py:52-78)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1, bias=True,
                 w_scale=1.0, b_scale=1.0):
        super().__init__(in_channels, out_channels, kernel_size, stride=stride, padding=padding, dilation=dilation,
                         groups=groups, bias=bias)
        _scaled_init(self, in_channels * kernel_size * kernel_size, w_scale, b_scale)

    def _conv(self, t, weight, bias):
        return F.conv2d(t, weight, bias, stride=self.stride, padding=self.padding, dilation=self.dilation,
                        groups=self.groups)

    def forward(self, x=None, lower=None, upper=None):
        bias = None if self.bias is None else self.bias * self.b_scale
        if x is not None:
            x = self._conv(x, self.weight * self.w_scale, bias)
        if lower is not None and upper is not None:
            c2, r2 = _center_radius(lower, upper)
            mid = self._conv(c2, self.weight * (self.w_scale / 2), bias)
            spread = self._conv(r2, self.weight.abs() * (self.w_scale / 2), None)
            lower, upper = mid - spread, mid + spread
        return x, lower, upper


class BoundTanh(nn.Tanh):
    """reference: basic_modules.py:17-19"""

    def forward(self, x=None, lower=None, upper=None):
        return apply_if_not_none((x, lower, upper), torch.tanh)


class BoundReLU(nn.ReLU):
    """Monotone activation: bounds pass through it unchanged in role (reference: basic_modules.py:12-14)."""

    def forward(self, x=None, lower=None, upper=None):
        return apply_if_not_none((x, lower, upper), F.relu)
