"""Autograd front-end of the L_p-distance operator (drop-in for the reference's core/norm_dist.py).

Public names, argument orders, defaults and return types follow the reference:
`norm_dist(input, weight, p, groups=1, use_custom_cuda_func=True, tag=None)` (core/norm_dist.py:94-104) and
`bound_inf_dist(x_lower, x_upper, weight, groups=1, use_custom_cuda_func=True, tag=None)` (:107-121), backed by the
autograd functions `NormDistF` (:6-51) and `BoundInfDistF` (:54-91).

Shapes: input [B, CI, HW], weight [CO, CI // groups], result [B, CO, HW].
`use_custom_cuda_func=False` selects the same broadcast tensor formulas the reference offers as its non-kernel
branch; it exists for API compatibility and is differentiable through torch autograd.
"""
import math

import torch

from . import _C

INF = float("inf")


def _new_output(x, weight):
    return torch.empty(x.size(0), weight.size(0), x.size(2), device=x.device, dtype=torch.float32)


class NormDistF(torch.autograd.Function):
    """forward(x, weight, group, p, need_grad, tag) -> output; gradients for x and weight."""

    @staticmethod
    def forward(ctx, x, weight, group, p, need_grad, tag):
        assert weight.size(1) * group == x.size(1)
        ctx.group, ctx.p, ctx.tag = group, p, tag
        out = _new_output(x, weight)
        if math.isinf(p):
            if need_grad:
                pos = torch.empty_like(out, dtype=torch.int32)
                _C.inf_dist_forward(x, weight, out, pos, group)
                ctx.save_for_backward(x, weight, pos)
            else:
                _C.inf_dist_forward_nograd(x, weight, out, group)
        elif p > 0:
            _C.norm_dist_forward(x, weight, out, group, p)
            ctx.save_for_backward(x, weight, out)
        else:
            raise NotImplementedError
        return out

    @staticmethod
    def backward(ctx, grad_output):
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        grad_output = grad_output.contiguous()
        grad_x = grad_w = None
        if math.isinf(ctx.p):
            x, weight, pos = ctx.saved_tensors
            if want_w:  # the fused kernel always produces both
                grad_x, grad_w = torch.empty_like(x), torch.empty_like(weight)
                _C.inf_dist_backward_input_weight(grad_output, pos, grad_x, grad_w, ctx.group)
            elif want_x:
                grad_x = torch.empty_like(x)
                _C.inf_dist_backward_input(grad_output, pos, grad_x, ctx.group)
        else:
            x, weight, out = ctx.saved_tensors
            if want_w:
                grad_x, grad_w = torch.empty_like(x), torch.empty_like(weight)
                _C.norm_dist_backward_input_weight(grad_output, x, weight, out, grad_x, grad_w, ctx.group, ctx.p)
            elif want_x:
                grad_x = torch.empty_like(x)
                _C.norm_dist_backward_input(grad_output, x, weight, out, grad_x, ctx.group, ctx.p)
        if not want_x:
            grad_x = None
        return grad_x, grad_w, None, None, None, None, None


class BoundInfDistF(torch.autograd.Function):
    """forward(x_lower, x_upper, weight, group, need_grad, tag) -> (y_lower, y_upper)."""

    @staticmethod
    def forward(ctx, x_lower, x_upper, weight, group, need_grad, tag):
        assert x_lower.size() == x_upper.size()
        assert weight.size(1) * group == x_lower.size(1)
        ctx.group, ctx.tag = group, tag
        y_lower = _new_output(x_lower, weight)
        y_upper = torch.empty_like(y_lower)
        if need_grad:
            pos_lower = torch.empty_like(y_lower, dtype=torch.int32)
            pos_upper = torch.empty_like(pos_lower)
            _C.bound_inf_dist_forward(x_lower, x_upper, weight, y_lower, y_upper, pos_lower, pos_upper, group)
            ctx.save_for_backward(x_lower, x_upper, weight, pos_lower, pos_upper)
        else:
            _C.bound_inf_dist_forward_nograd(x_lower, x_upper, weight, y_lower, y_upper, group)
        return y_lower, y_upper

    @staticmethod
    def backward(ctx, grad_y_lower, grad_y_upper):
        want_l, want_u, want_w = ctx.needs_input_grad[:3]
        grad_y_lower = grad_y_lower.contiguous()
        grad_y_upper = grad_y_upper.contiguous()
        x_lower, x_upper, weight, pos_lower, pos_upper = ctx.saved_tensors
        # zero-initialised like the reference: the input-only kernel runs only when both inputs want gradients
        grad_l, grad_u, grad_w = torch.zeros_like(x_lower), torch.zeros_like(x_upper), None
        if want_w:
            grad_w = torch.zeros_like(weight)
            _C.bound_inf_dist_backward_input_weight(grad_y_lower, grad_y_upper, pos_lower, pos_upper,
                                                    grad_l, grad_u, grad_w, ctx.group)
        elif want_l and want_u:
            _C.bound_inf_dist_backward_input(grad_y_lower, grad_y_upper, pos_lower, pos_upper,
                                             grad_l, grad_u, ctx.group)
        return (grad_l if want_l else None, grad_u if want_u else None, grad_w, None, None, None, None, None)


class UnfoldF(torch.autograd.Function):
    """Patch extraction [B, C, H, W] -> [B, C*kh*kw, OH*OW] and its adjoint, one kernel launch each."""

    @staticmethod
    def forward(ctx, x, kernel_size, dilation, padding, stride):
        ctx.args = (kernel_size, dilation, padding, stride)
        ctx.in_shape = x.shape
        geo, (oh, ow) = _C.unfold_geometry(x.shape, *ctx.args)
        out = torch.empty(geo[0], geo[1] * geo[4] * geo[5], oh * ow, device=x.device, dtype=torch.float32)
        _C.unfold_forward(x, out, *ctx.args)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        grad_x = torch.empty(ctx.in_shape, device=grad_output.device, dtype=torch.float32)
        _C.unfold_backward(grad_output.contiguous(), grad_x, *ctx.args)
        return grad_x, None, None, None, None


def unfold(x, kernel_size, dilation=1, padding=0, stride=1):
    """torch.nn.functional.unfold for the convolutional distance layer (reference: core/modules/norm_dist.py:93-102
    calls F.unfold).  fp32 tensors on the GPU go through the library's kernels; anything else is left to torch, as
    in the reference."""
    if x.is_cuda and x.dtype == torch.float32 and x.dim() == 4:
        return UnfoldF.apply(x.contiguous(), kernel_size, dilation, padding, stride)
    return torch.nn.functional.unfold(x, kernel_size, dilation, padding, stride)


class ConvInfDistF(torch.autograd.Function):
    """Infinity distance of a convolutional layer on images [B, C, H, W]: NormDistF on the unfolded input, without the
    unfolded tensor (forward) or its gradient (backward) ever being written."""

    @staticmethod
    def forward(ctx, x, weight, group, geometry, tag):
        ctx.group, ctx.geometry, ctx.tag = group, geometry, tag
        ctx.in_shape = x.shape
        _, (oh, ow) = _C.unfold_geometry(x.shape, *geometry)
        out = torch.empty(x.size(0), weight.size(0), oh * ow, device=x.device, dtype=torch.float32)
        pos = torch.empty_like(out, dtype=torch.int32)
        _C.conv_inf_dist_forward(x, weight, out, pos, group, *geometry)
        ctx.save_for_backward(weight, pos)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        weight, pos = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_x = grad_w = None
        if want_w:
            grad_x = torch.empty(ctx.in_shape, device=grad_output.device, dtype=torch.float32)
            grad_w = torch.empty_like(weight)
            _C.conv_inf_dist_backward_input_weight(grad_output, pos, grad_x, grad_w, ctx.group, *ctx.geometry)
        elif want_x:
            grad_x = torch.empty(ctx.in_shape, device=grad_output.device, dtype=torch.float32)
            _C.conv_inf_dist_backward_input(grad_output, pos, grad_x, weight.shape, ctx.group, *ctx.geometry)
        return (grad_x if want_x else None), grad_w, None, None, None


class ConvNormDistF(torch.autograd.Function):
    """Finite-p distance of a convolutional layer on images [B, C, H, W]: NormDistF on the unfolded input without the
    unfolded tensor: the forward extracts the patches while loading its tiles and keeps the image (not its nine
    times larger patches) for the backward, which writes the patches once in the layout its kernel reads."""

    @staticmethod
    def forward(ctx, x, weight, group, p, geometry, tag):
        ctx.group, ctx.p, ctx.geometry, ctx.tag = group, p, geometry, tag
        _, (oh, ow) = _C.unfold_geometry(x.shape, *geometry)
        out = torch.empty(x.size(0), weight.size(0), oh * ow, device=x.device, dtype=torch.float32)
        _C.conv_norm_dist_forward(x, weight, out, group, p, *geometry)
        ctx.save_for_backward(x, weight, out)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        x, weight, out = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_x = grad_w = None
        if want_w:
            grad_x, grad_w = torch.empty_like(x), torch.empty_like(weight)
            _C.conv_norm_dist_backward_input_weight(grad_output, x, weight, out, grad_x, grad_w, ctx.group, ctx.p,
                                                    *ctx.geometry)
        elif want_x:
            grad_x = torch.empty_like(x)
            _C.conv_norm_dist_backward_input(grad_output, x, weight, out, grad_x, ctx.group, ctx.p, *ctx.geometry)
        return (grad_x if want_x else None), grad_w, None, None, None, None


class ConvBoundInfDistF(torch.autograd.Function):
    """Interval bounds of a convolutional layer on image boxes: BoundInfDistF on the unfolded bounds, fused like
    ConvInfDistF."""

    @staticmethod
    def forward(ctx, x_lower, x_upper, weight, group, geometry, tag):
        assert x_lower.size() == x_upper.size()
        ctx.group, ctx.geometry, ctx.tag = group, geometry, tag
        ctx.in_shape = x_lower.shape
        _, (oh, ow) = _C.unfold_geometry(x_lower.shape, *geometry)
        y_lower = torch.empty(x_lower.size(0), weight.size(0), oh * ow, device=x_lower.device, dtype=torch.float32)
        y_upper = torch.empty_like(y_lower)
        pos_lower = torch.empty_like(y_lower, dtype=torch.int32)
        pos_upper = torch.empty_like(pos_lower)
        _C.conv_bound_inf_dist_forward(x_lower, x_upper, weight, y_lower, y_upper, pos_lower, pos_upper, group, *geometry)
        ctx.save_for_backward(weight, pos_lower, pos_upper)
        return y_lower, y_upper

    @staticmethod
    def backward(ctx, grad_y_lower, grad_y_upper):
        want_l, want_u, want_w = ctx.needs_input_grad[:3]
        weight, pos_lower, pos_upper = ctx.saved_tensors
        grad_y_lower, grad_y_upper = grad_y_lower.contiguous(), grad_y_upper.contiguous()
        dev = grad_y_lower.device
        grad_l = grad_u = grad_w = None
        if want_w:
            grad_l = torch.empty(ctx.in_shape, device=dev, dtype=torch.float32)
            grad_u, grad_w = torch.empty_like(grad_l), torch.empty_like(weight)
            _C.conv_bound_inf_dist_backward_input_weight(grad_y_lower, grad_y_upper, pos_lower, pos_upper, grad_l, grad_u,
                                                         grad_w, ctx.group, *ctx.geometry)
        elif want_l and want_u:
            grad_l = torch.empty(ctx.in_shape, device=dev, dtype=torch.float32)
            grad_u = torch.empty_like(grad_l)
            _C.conv_bound_inf_dist_backward_input(grad_y_lower, grad_y_upper, pos_lower, pos_upper, grad_l, grad_u,
                                                  weight.shape, ctx.group, *ctx.geometry)
        else:  # like BoundInfDistF: the input-only kernel runs only when both inputs want gradients
            grad_l = torch.zeros(ctx.in_shape, device=dev, dtype=torch.float32)
            grad_u = torch.zeros_like(grad_l)
        return (grad_l if want_l else None), (grad_u if want_u else None), grad_w, None, None, None


def _fused_conv_ok(*tensors):
    return all(t.is_cuda and t.dtype == torch.float32 and t.dim() == 4 for t in tensors)


def _empty_batch(shape, count, *tensors):
    """An empty batch.  The reference's kernels are launched over no rows then and leave an empty output, and its
    backward clears grad_weight before a launch that does nothing (core/cuda/norm_dist_cuda.cu:515-520, 602-604); the
    C ABI here refuses empty shapes, so the empty outputs are formed on the host, tied to the inputs and the weight
    so that these receive zero gradients."""
    tie = sum(t.sum() * 0 for t in tensors)
    outs = tuple(tensors[0].new_zeros(shape) + tie for _ in range(count))
    return outs[0] if count == 1 else outs


def conv_norm_dist(input, weight, p, kernel_size, dilation=1, padding=0, stride=1, groups=1, tag=None):
    """norm_dist(unfold(input), weight, p, groups) for images [B, C, H, W] (what the reference's NormDistConv
    computes, core/modules/norm_dist.py:93-102).  At p = inf the kernels extract the patches while they load their
    tiles and scatter the gradient straight into the image: neither the unfolded tensor nor its gradient is ever
    written; values and arg-max codes are bit-identical.  Finite p works on the image too: the forward extracts the
    patches on the fly, the backward writes them once as rows for its kernel and folds the gradient rows back."""
    if input.size(0) == 0:
        _, (oh, ow) = _C.unfold_geometry(input.shape, kernel_size, dilation, padding, stride)
        return _empty_batch((0, weight.size(0), oh * ow), 1, input, weight)
    need_grad = torch.is_grad_enabled() and (input.requires_grad or weight.requires_grad)
    if not math.isinf(p) and _fused_conv_ok(input) and weight.is_cuda:
        if p <= 0:
            raise ValueError("p must be positive")
        geometry = (kernel_size, dilation, padding, stride)
        if need_grad:
            return ConvNormDistF.apply(input.contiguous(), weight.contiguous(), groups, float(p), geometry, tag)
        _, (oh, ow) = _C.unfold_geometry(input.shape, *geometry)
        out = torch.empty(input.size(0), weight.size(0), oh * ow, device=input.device, dtype=torch.float32)
        _C.conv_norm_dist_forward(input.contiguous(), weight.contiguous(), out, groups, float(p), *geometry)
        return out
    if math.isinf(p) and _fused_conv_ok(input):
        geometry = (kernel_size, dilation, padding, stride)
        if need_grad:
            return ConvInfDistF.apply(input.contiguous(), weight.contiguous(), groups, geometry, tag)
        _, (oh, ow) = _C.unfold_geometry(input.shape, *geometry)
        out = torch.empty(input.size(0), weight.size(0), oh * ow, device=input.device, dtype=torch.float32)
        _C.conv_inf_dist_forward_nograd(input.contiguous(), weight.contiguous(), out, groups, *geometry)
        return out
    return norm_dist(unfold(input, kernel_size, dilation, padding, stride), weight, p, groups, tag=tag)


def conv_bound_inf_dist(x_lower, x_upper, weight, kernel_size, dilation=1, padding=0, stride=1, groups=1, tag=None):
    """bound_inf_dist(unfold(x_lower), unfold(x_upper), weight, groups) for image boxes [B, C, H, W]; fused like
    conv_norm_dist."""
    if x_lower.size(0) == 0:
        _, (oh, ow) = _C.unfold_geometry(x_lower.shape, kernel_size, dilation, padding, stride)
        return _empty_batch((0, weight.size(0), oh * ow), 2, x_lower, x_upper, weight)
    need_grad = torch.is_grad_enabled() and (x_lower.requires_grad or x_upper.requires_grad or weight.requires_grad)
    if need_grad and _fused_conv_ok(x_lower, x_upper):
        return ConvBoundInfDistF.apply(x_lower.contiguous(), x_upper.contiguous(), weight.contiguous(), groups,
                                       (kernel_size, dilation, padding, stride), tag)
    if _fused_conv_ok(x_lower, x_upper):
        assert x_lower.size() == x_upper.size()
        _, (oh, ow) = _C.unfold_geometry(x_lower.shape, kernel_size, dilation, padding, stride)
        y_lower = torch.empty(x_lower.size(0), weight.size(0), oh * ow, device=x_lower.device, dtype=torch.float32)
        y_upper = torch.empty_like(y_lower)
        _C.conv_bound_inf_dist_forward_nograd(x_lower.contiguous(), x_upper.contiguous(), weight.contiguous(), y_lower,
                                              y_upper, groups, kernel_size, dilation, padding, stride)
        return y_lower, y_upper
    return bound_inf_dist(unfold(x_lower, kernel_size, dilation, padding, stride),
                          unfold(x_upper, kernel_size, dilation, padding, stride), weight, groups, tag=tag)


class WeightCache:
    """The p = inf forwards' pre-pass over a layer's weights, taken once by `freeze(weight, groups)` and handed to the
    *_cached entry points until `drop()`.  Strictly opt-in (the layers' `freeze_weights()`): while frozen the caller
    promises that the weights keep their values.  Updates that torch can see (a new parameter tensor, another
    storage address, an advanced version counter, another shape or device) still redo the pre-pass, but writes
    through `weight.data` advance no counter and cannot be seen: after such a write call `freeze` again or `drop`.
    Non-contiguous weights are never cached (their contiguous copy is a new tensor on every call).  No counterpart
    in the reference, which keeps no state between calls."""

    def __init__(self):
        self._key, self._buffer, self.frozen = None, None, False

    @staticmethod
    def _key_of(weight, groups):
        return (weight.data_ptr(), weight._version, tuple(weight.shape), groups, weight.device)

    def freeze(self, weight, groups):
        """Take (or retake) the pre-pass of `weight` as it is now."""
        self.drop()
        if weight.is_cuda and weight.dtype == torch.float32 and weight.is_contiguous():
            self._buffer = _C.weight_cache(weight.detach(), groups)
            self._key = self._key_of(weight, groups)
            self.frozen = True
        return self.frozen

    def drop(self):
        self._key, self._buffer, self.frozen = None, None, False

    def get(self, weight, groups):
        """The kept buffer for `weight`, retaken when torch shows that the weights changed; None when not frozen or
        when `weight` cannot be cached."""
        if not self.frozen:
            return None
        if not (weight.is_cuda and weight.is_contiguous()):
            return None
        if self._key_of(weight, groups) != self._key:
            self.freeze(weight, groups)
        return self._buffer


def inf_dist_nograd(x, weight, groups=1, cache=None):
    """The infinity distance without gradients, optionally with the weights' pre-pass taken from `cache`
    (WeightCache)."""
    if x.size(0) == 0:
        return _new_output(x, weight)
    buffer = cache.get(weight, groups) if cache is not None else None
    x, weight = x.contiguous(), weight.contiguous()
    y = _new_output(x, weight)
    if buffer is not None:
        _C.inf_dist_forward_nograd_cached(x, weight, buffer, y, groups)
    else:
        _C.inf_dist_forward_nograd(x, weight, y, groups)
    return y


def inf_dist_with_bounds(x, x_lower, x_upper, weight, groups=1, tag=None, cache=None):
    """(y, y_lower, y_upper): the infinity distance of x and the interval bounds of the box (x_lower, x_upper) against
    the same weights: what a layer computes under certification (reference: core/modules/norm_dist.py:30-34, two
    operator calls).  Without gradients the two run as one library call that shares the pre-pass over the weights;
    with gradients they are the two autograd operators."""
    tensors = (x, x_lower, x_upper, weight)
    if (x.size(0) > 0 and all(t.is_cuda and t.dtype == torch.float32 for t in tensors)
            and not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors))):
        buffer = cache.get(weight, groups) if cache is not None else None
        x, x_lower, x_upper, weight = (t.contiguous() for t in tensors)
        y = _new_output(x, weight)
        y_lower, y_upper = torch.empty_like(y), torch.empty_like(y)
        if buffer is not None:
            _C.inf_and_bound_forward_nograd_cached(x, x_lower, x_upper, weight, buffer, y, y_lower, y_upper, groups)
        else:
            _C.inf_and_bound_forward_nograd(x, x_lower, x_upper, weight, y, y_lower, y_upper, groups)
        return y, y_lower, y_upper
    y = norm_dist(x, weight, INF, groups, tag=tag)
    y_lower, y_upper = bound_inf_dist(x_lower, x_upper, weight, groups, tag=tag)
    return y, y_lower, y_upper


class MeanShiftBiasF(torch.autograd.Function):
    """What follows the operator in every layer (reference: core/modules/norm_dist.py:35-38 and
    core/modules/basic_modules.py:121-132), as one fused call: y* = t* - mean + bias1 + bias2 for t* in
    (x, lower, upper), with mean the batch mean of x over (batch, position) in training (differentiable, also folded
    into running_mean) or running_mean itself in evaluation; use_mean=False leaves the mean out (bias only).
    Returns (y, y_lower, y_upper) with None where the input was None."""

    @staticmethod
    def forward(ctx, x, lower, upper, running_mean, momentum, training, use_mean, bias1, bias2):
        batch_mean = bool(training and use_mean)
        if batch_mean:
            assert x is not None, 'Currently not supported'  # as the reference (core/modules/basic_modules.py:123)
        x, lower, upper = (None if t is None else t.contiguous() for t in (x, lower, upper))
        lead = next(t for t in (x, lower, upper) if t is not None)
        C = lead.size(1)
        ys = tuple(None if t is None else torch.empty_like(t) for t in (x, lower, upper))
        mean_out = torch.empty(C, device=lead.device, dtype=torch.float32) if batch_mean else None
        _C.mean_shift_forward(x, lower, upper, batch_mean, momentum, running_mean if use_mean else None,
                              None if bias1 is None else bias1.detach(), None if bias2 is None else bias2.detach(),
                              mean_out, *ys)
        ctx.batch_mean = batch_mean
        ctx.channels = C
        ctx.bias_grad = (bias1 is not None and bias1.requires_grad, bias2 is not None and bias2.requires_grad)
        ctx.set_materialize_grads(False)
        return ys

    @staticmethod
    def backward(ctx, gy, gyl, gyu):
        gy, gyl, gyu = (None if g is None else g.contiguous() for g in (gy, gyl, gyu))
        lead = next((g for g in (gy, gyl, gyu) if g is not None), None)
        if lead is None:
            return (None,) * 9
        want_cols = any(ctx.bias_grad)
        new = lambda: torch.empty(ctx.channels, device=lead.device, dtype=torch.float32)
        colsum = new() if want_cols else None
        gx = gy
        if ctx.batch_mean and ctx.needs_input_grad[0]:
            if gy is None:
                gy = torch.zeros_like(lead)  # only the bounds were used: grad_x is minus the mean of their gradients
            gx = torch.empty_like(gy)
            _C.mean_shift_backward(gy, gyl, gyu, True, gx, colsum, new())
        elif want_cols:
            _C.mean_shift_backward(gy, gyl, gyu, False, None, colsum, new())
        return (gx, gyl, gyu, None, None, None, None,
                colsum if ctx.bias_grad[0] else None, colsum if ctx.bias_grad[1] else None)


def mean_shift_bias(x, lower, upper, running_mean, momentum, training, bias1=None, bias2=None):
    """Fused mean shift (running_mean is not None) and bias add for CUDA tensors [B, C, HW]; see MeanShiftBiasF."""
    return MeanShiftBiasF.apply(x, lower, upper, running_mean, momentum, training, running_mean is not None, bias1, bias2)


def _grouped(t, groups):
    return t.view(t.size(0), groups, 1, -1, t.size(2))  # [B, G, 1, CI/G, HW]


def norm_dist(input, weight, p, groups=1, use_custom_cuda_func=True, tag=None):
    if use_custom_cuda_func and input.size(0) == 0:
        return _empty_batch((0, weight.size(0), input.size(2)), 1, input, weight)
    if use_custom_cuda_func:
        need_grad = torch.is_grad_enabled() and (input.requires_grad or weight.requires_grad)
        return NormDistF.apply(input, weight, groups, p, need_grad, tag)
    diff = _grouped(input, groups) - weight.view(groups, -1, weight.size(-1), 1)
    with torch.no_grad():
        scale = torch.norm(diff, dim=3, p=INF, keepdim=True)
    y = torch.norm(diff / scale, dim=3, p=p, keepdim=True) * scale
    return y.view(y.size(0), -1, y.size(-1))


def bound_inf_dist(x_lower, x_upper, weight, groups=1, use_custom_cuda_func=True, tag=None):
    if use_custom_cuda_func and x_lower.size(0) == 0:
        return _empty_batch((0, weight.size(0), x_lower.size(2)), 2, x_lower, x_upper, weight)
    if use_custom_cuda_func:
        need_grad = torch.is_grad_enabled() and (x_lower.requires_grad or x_upper.requires_grad or weight.requires_grad)
        return BoundInfDistF.apply(x_lower, x_upper, weight, groups, need_grad, tag)
    w = weight.view(groups, -1, weight.size(-1), 1)
    below = w - _grouped(x_lower, groups)
    above = _grouped(x_upper, groups) - w
    far = torch.maximum(below, above).clamp(min=1e-10)
    near = torch.minimum(below, above).clamp(max=-1e-10)
    y_upper = torch.norm(far, dim=3, p=INF, keepdim=True)
    y_lower = torch.norm(-near, dim=3, p=INF, keepdim=True)
    shape = (x_lower.size(0), -1, x_lower.size(-1))
    return y_lower.view(shape), y_upper.view(shape)


class WorstMarginF(torch.autograd.Function):
    """Worst-case margins of the logits -x against the target class (reference: ell_inf_models.py:41-46, a dozen
    torch primitives there): margin[b, c] = (upper[b, t_b] - lower[b, c]) / (2 eps), 0 at the target; without
    bounds lower / upper = x -/+ eps.  One launch each way."""

    @staticmethod
    def forward(ctx, x, lower, upper, targets, eps):
        lead = x if lower is None else lower
        margin = torch.empty_like(lead)
        _C.margin_forward(None if lower is not None else x, lower, upper, targets, eps, margin)
        ctx.save_for_backward(targets)
        ctx.eps, ctx.bounds = eps, lower is not None
        return margin

    @staticmethod
    def backward(ctx, grad_margin):
        targets, = ctx.saved_tensors
        grad_margin = grad_margin.contiguous()
        if ctx.bounds:
            grad_lower, grad_upper = torch.empty_like(grad_margin), torch.empty_like(grad_margin)
            _C.margin_backward(grad_margin, targets, ctx.eps, None, grad_lower, grad_upper)
            return None, grad_lower, grad_upper, None, None
        grad_x = torch.empty_like(grad_margin)
        _C.margin_backward(grad_margin, targets, ctx.eps, grad_x, None, None)
        return grad_x, None, None, None, None


def worst_margin(x, lower, upper, targets, eps):
    """Margins for `hinge`; the fused kernels on CUDA float32 [B, C] tensors, torch primitives otherwise."""
    lead = x if lower is None else lower
    if (lead.is_cuda and lead.dtype == torch.float32 and lead.dim() == 2 and eps > 0
            and (lower is None) == (upper is None) and targets.dtype == torch.int64):
        args = [None if t is None else t.contiguous() for t in (x, lower, upper)]
        return WorstMarginF.apply(args[0], args[1], args[2], targets.contiguous(), float(eps))
    if lower is None:
        lower, upper = x - eps, x + eps
    idx = targets.view(-1, 1)
    return (torch.gather(upper, 1, idx) - lower).scatter(1, idx, 0) / (2 * eps)


class HingeF(torch.autograd.Function):
    """(1 - mix) * mean_b max_c relu(m) + mix * mean relu(m) on the margins (reference: main.py:304-310)."""

    @staticmethod
    def forward(ctx, margin, mix):
        loss = torch.empty(1, device=margin.device, dtype=torch.float32)
        argmax = torch.empty(margin.size(0), device=margin.device, dtype=torch.int32)
        _C.hinge_forward(margin, mix, loss, argmax)
        ctx.save_for_backward(margin, argmax)
        ctx.mix = mix
        return loss.view(())

    @staticmethod
    def backward(ctx, grad_loss):
        margin, argmax = ctx.saved_tensors
        grad_margin = torch.empty_like(margin)
        _C.hinge_backward(margin, argmax, grad_loss.contiguous().view(1).float(), ctx.mix, grad_margin)
        return grad_margin, None


def hinge_loss(margin, mix):
    if margin.is_cuda and margin.dtype == torch.float32 and margin.dim() == 2:
        return HingeF.apply(margin.contiguous(), float(mix))
    res = margin.clamp(min=0)
    return (1 - mix) * res.max(dim=1)[0].mean() + mix * res.mean()
