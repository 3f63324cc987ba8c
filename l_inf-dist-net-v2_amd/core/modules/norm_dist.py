"""L_p-distance layers (drop-in for the reference's core/modules/norm_dist.py): `NormDistBase`, the fully-connected
`NormDist` and the convolutional `NormDistConv`.  Constructor arguments, parameter / buffer names (`weight`, `bias`,
`mean_shift.running_mean`) and the (x, lower, upper) calling convention are the reference's, so its checkpoints load.
"""
import math

import torch
import torch.nn as nn

from core.norm_dist import (norm_dist, bound_inf_dist, conv_norm_dist, conv_bound_inf_dist, mean_shift_bias,
                            inf_dist_with_bounds, inf_dist_nograd, WeightCache)
from .basic_modules import MeanShift, apply_if_not_none


class NormDistBase(nn.Module):
    """out[b, co, hw] = || x[b, group(co), :, hw] - weight[co, :] ||_p, then optional mean shift and bias.
    Inputs are [B, C, H*W] (reference: core/modules/norm_dist.py:13-39)."""

    def __init__(self, in_features, out_features, p=float('inf'), groups=1, bias=True, std=1.0, mean_shift=True):
        super().__init__()
        assert in_features % groups == 0
        assert out_features % groups == 0
        self.weight = nn.Parameter(torch.randn(out_features, in_features // groups) * std)
        self.groups = groups
        self.p = p
        self.mean_shift = MeanShift(out_channels=out_features, affine=False) if mean_shift else None
        self.bias = nn.Parameter(torch.zeros(out_features)) if bias else None
        NormDistBase.tag = getattr(NormDistBase, 'tag', 0) + 1
        self.tag = NormDistBase.tag
        self._weight_cache = WeightCache()  # plain attribute: not a parameter or buffer, never in the state dict

    def freeze_weights(self):
        """Opt in to keeping the p = inf forwards' pre-pass over the weights between calls (evaluation,
        certification, serving; no counterpart in the reference).  Takes the pre-pass now; from here on the caller
        promises that the weights keep their values until `unfreeze_weights()`.  `train()`, `load_state_dict` and
        moves between devices unfreeze; in-place updates that advance the parameter's version counter redo the
        pre-pass; writes through `weight.data` are invisible to torch: call `freeze_weights()` again after them.
        Returns True when the weights could be cached (contiguous float32 on the GPU)."""
        return self._weight_cache.freeze(self.weight, self.groups)

    def unfreeze_weights(self):
        self._weight_cache.drop()

    def train(self, mode=True):
        if mode:
            self._weight_cache.drop()
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self._weight_cache.drop()
        return super()._load_from_state_dict(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self._weight_cache.drop()
        return super()._apply(fn, *args, **kwargs)

    def forward(self, x=None, lower=None, upper=None):
        # kept pre-pass of the weights: only after freeze_weights(), only in evaluation without gradients
        use = (self._weight_cache.frozen and not self.training and not torch.is_grad_enabled() and math.isinf(self.p)
               and self.weight.is_cuda)
        cache = self._weight_cache if use else None
        if x is not None and lower is not None and upper is not None and math.isinf(self.p) and x.is_cuda:
            # the distance and its bounds against the same weights: one call (shares the pre-pass over the weights)
            x, lower, upper = inf_dist_with_bounds(x, lower, upper, self.weight, self.groups, tag=self.tag, cache=cache)
            return self._shift_and_bias(x, lower, upper)
        if x is not None:
            if cache is not None and x.is_cuda and x.dtype == torch.float32:
                x = inf_dist_nograd(x, self.weight, self.groups, cache=cache)
            else:
                x = norm_dist(x, self.weight, self.p, self.groups, tag=self.tag)
        if lower is not None and upper is not None:
            assert math.isinf(self.p)  # interval propagation exists for the infinity distance only
            lower, upper = bound_inf_dist(lower, upper, self.weight, self.groups, tag=self.tag)
        return self._shift_and_bias(x, lower, upper)

    def _shift_and_bias(self, x, lower, upper):
        lead = next((t for t in (x, lower, upper) if t is not None), None)
        if lead is not None and lead.is_cuda and lead.dtype == torch.float32 and \
                (self.mean_shift is not None or self.bias is not None):
            # one fused call for the mean shift (with its moving average) and both biases
            ms = self.mean_shift
            return mean_shift_bias(x, lower, upper, ms.running_mean if ms is not None else None,
                                   ms.momentum if ms is not None else 0.0, ms.training if ms is not None else False,
                                   ms.bias if ms is not None else None, self.bias)
        if self.mean_shift is not None:
            x, lower, upper = self.mean_shift(x, lower, upper)
        if self.bias is not None:
            b = self.bias.view(1, -1, 1)
            x, lower, upper = apply_if_not_none((x, lower, upper), lambda t: t + b)
        return x, lower, upper


def freeze_weights(model):
    """`freeze_weights()` on every distance layer of `model`; returns how many layers now keep their pre-pass."""
    return sum(bool(m.freeze_weights()) for m in model.modules() if isinstance(m, NormDistBase))


def unfreeze_weights(model):
    for m in model.modules():
        if isinstance(m, NormDistBase):
            m.unfreeze_weights()


class NormDistConv(NormDistBase):
    """Convolutional distance layer on [B, C, H, W]: patches are unfolded to [B, C*kh*kw, H'*W'] and fed to the
    same operator (reference: core/modules/norm_dist.py:66-110)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, identity_val=None, **kwargs):
        if isinstance(kernel_size, int):
            kernel_size = (kernel_size, kernel_size)
        assert in_channels % groups == 0
        super().__init__(in_channels * kernel_size[0] * kernel_size[1], out_channels, groups=groups, bias=bias, **kwargs)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride, self.padding, self.dilation = kernel_size, stride, padding, dilation
        if identity_val is not None and in_channels <= out_channels:
            # -identity_val at the centre tap of the wrapped diagonal channel
            co = torch.arange(out_channels)
            with torch.no_grad():
                self.weight.view(out_channels, -1, *kernel_size)[
                    co, co % (in_channels // groups), kernel_size[0] // 2, kernel_size[1] // 2] = -identity_val

    def forward(self, x=None, lower=None, upper=None):
        # the operators take the images: they unfold them when a gradient is wanted and extract the patches inside
        # the kernel when it is not (evaluation, certification)
        h = w = 0
        geometry = (self.kernel_size, self.dilation, self.padding, self.stride)
        if x is not None:
            h, w = x.size(2), x.size(3)
            x = conv_norm_dist(x, self.weight, self.p, *geometry, groups=self.groups, tag=self.tag)
        if lower is not None and upper is not None:
            assert math.isinf(self.p)
            h, w = lower.size(2), lower.size(3)
            lower, upper = conv_bound_inf_dist(lower, upper, self.weight, *geometry, groups=self.groups, tag=self.tag)
        x, lower, upper = self._shift_and_bias(x, lower, upper)
        # output size as the reference computes it (dilation is not accounted for there either)
        h, w = [(size + 2 * self.padding - k) // self.stride + 1 for size, k in zip((h, w), self.kernel_size)]
        return apply_if_not_none((x, lower, upper), lambda t: t.view(t.size(0), -1, h, w))

    def extra_repr(self):
        text = ['%d, %d' % (self.in_channels, self.out_channels), 'kernel_size=%s' % (self.kernel_size,),
                'stride=%s' % (self.stride,)]
        # non-default settings only
        for name, default in (('padding', 0), ('dilation', 1), ('groups', 1)):
            if getattr(self, name) != default:
                text.append('%s=%s' % (name, getattr(self, name)))
        if self.bias is None:
            text.append('bias=False')
        return ', '.join(text)


class NormDist(NormDistBase):
    """Fully-connected distance layer on [B, C] tensors (reference: core/modules/norm_dist.py:42-63).
    `identity_val` plants -identity_val on the wrapped diagonal when the layer does not shrink."""

    def __init__(self, in_features, out_features, groups=1, bias=True, identity_val=None, **kwargs):
        super().__init__(in_features, out_features, groups=groups, bias=bias, **kwargs)
        self.in_features = in_features
        self.out_features = out_features
        if identity_val is not None and in_features <= out_features:
            rows = torch.arange(out_features)
            with torch.no_grad():
                self.weight[rows, rows % (in_features // groups)] = -identity_val

    def forward(self, x=None, lower=None, upper=None):
        triple = apply_if_not_none((x, lower, upper), lambda t: t.unsqueeze(-1))
        triple = super().forward(*triple)
        return apply_if_not_none(triple, lambda t: t.squeeze(-1))

    def extra_repr(self):
        shown = [('in_features', self.in_features), ('out_features', self.out_features), ('bias', self.bias is not None)]
        if self.groups != 1:
            shown.append(('groups', self.groups))
        return ', '.join('%s=%s' % item for item in shown)
