"""The fused mean shift + bias of the distance layers (ndist_mean_shift_forward / _backward) against the reference's
own formulas (core/modules/basic_modules.py:121-132, core/modules/norm_dist.py:35-38) evaluated by torch in float64:
y* = t* - (mean - bias_ms) + bias_layer with mean the batch mean of x over (batch, position) in training (EMA
updated: running = 0.9 running + 0.1 mean) or the running mean in evaluation."""
import numpy as np
import pytest
import torch

from util import rel_err

pytestmark = pytest.mark.gpu

SHAPES = [(512, 5120, 1), (37, 130, 1), (6, 10, 49), (5, 7, 64), (128, 128, 1024), (3, 4, 1)]


def _reference(x, lo, up, running, momentum, training, b1, b2):
    """float64 torch formulas of the reference, with autograd."""
    if training:
        mean = x.mean(dim=[0, 2])
        new_running = running * (1 - momentum) + mean.detach() * momentum
    else:
        mean, new_running = running, running
    shift = mean
    if b1 is not None:
        shift = shift - b1
    outs = [None if t is None else t - shift[None, :, None] for t in (x, lo, up)]
    if b2 is not None:
        outs = [None if t is None else t + b2[None, :, None] for t in outs]
    return outs, new_running


@pytest.mark.parametrize("training", [True, False])
@pytest.mark.parametrize("bounds", [False, True])
@pytest.mark.parametrize("B,C,HW", SHAPES)
def test_forward_and_backward(B, C, HW, bounds, training):
    from core.norm_dist import mean_shift_bias
    if B * C * HW > 3e7 and bounds:
        pytest.skip("one large case is enough")
    gen = torch.Generator().manual_seed(B + C + HW)
    x = torch.randn(B, C, HW, generator=gen) * 3 + 1
    lo, up = (x - 0.3, x + 0.2) if bounds else (None, None)
    running = torch.randn(C, generator=gen)
    b1, b2 = torch.randn(C, generator=gen), torch.randn(C, generator=gen)
    gys = [torch.randn(B, C, HW, generator=gen) for _ in range(3)]
    # float64 reference
    leaves64 = [None if t is None else t.double().requires_grad_(True) for t in (x, lo, up, b1, b2)]
    outs64, run64 = _reference(leaves64[0], leaves64[1], leaves64[2], running.double(), 0.1, training, leaves64[3], leaves64[4])
    sum(((o * g.double()).sum() for o, g in zip(outs64, gys) if o is not None)).backward()
    # fused
    leaves = [None if t is None else t.cuda().requires_grad_(True) for t in (x, lo, up, b1, b2)]
    run = running.cuda()
    outs = mean_shift_bias(leaves[0], leaves[1], leaves[2], run, 0.1, training, leaves[3], leaves[4])
    sum(((o * g.cuda()).sum() for o, g in zip(outs, gys) if o is not None)).backward()
    for name, a, b in zip(("y", "y_lower", "y_upper"), outs, outs64):
        assert (a is None) == (b is None)
        if a is not None:
            assert rel_err(a.detach().cpu().numpy(), b.detach().numpy()) < 1e-6, name
    assert rel_err(run.cpu().numpy(), run64.numpy()) < 1e-6
    for name, a, b in zip(("grad_x", "grad_lower", "grad_upper", "grad_bias_ms", "grad_bias_layer"), leaves, leaves64):
        if a is not None:
            assert rel_err(a.grad.cpu().numpy(), b.grad.numpy()) < 1e-5, name
    # fixed summation order: a second run gives the same bits
    run2 = running.cuda()
    outs2 = mean_shift_bias(leaves[0].detach(), None if lo is None else leaves[1].detach(),
                            None if up is None else leaves[2].detach(), run2, 0.1, training, leaves[3].detach(),
                            leaves[4].detach())
    assert torch.equal(outs2[0], outs[0].detach()) and torch.equal(run2, run)


def test_bias_only_and_bounds_only():
    from core.norm_dist import mean_shift_bias
    gen = torch.Generator().manual_seed(3)
    lo = torch.randn(9, 12, 5, generator=gen).cuda().requires_grad_(True)
    up = (lo.detach() + 1).requires_grad_(True)
    bias = torch.randn(12, generator=gen).cuda().requires_grad_(True)
    y, yl, yu = mean_shift_bias(None, lo, up, None, 0.0, False, None, bias)  # last layer of the stack: bias, no shift
    assert y is None
    assert torch.allclose(yl, lo + bias[None, :, None]) and torch.allclose(yu, up + bias[None, :, None])
    (yl.sum() + 2 * yu.sum()).backward()
    assert torch.allclose(lo.grad, torch.ones_like(lo)) and torch.allclose(up.grad, 2 * torch.ones_like(up))
    assert torch.allclose(bias.grad, torch.full_like(bias, 3.0 * 9 * 5))


def test_layer_uses_the_fused_call_and_matches_the_torch_formulas():
    # NormDist (mean shift, no bias) and the last-layer form (bias, no shift) against the module's own torch path
    from core.modules import NormDist
    torch.manual_seed(8)
    for kw in ({"bias": False, "mean_shift": True}, {"bias": True, "mean_shift": False}):
        layer = NormDist(40, 24, **kw).cuda()
        layer.p = 8.0
        if layer.bias is not None:
            layer.bias.data.normal_()
        x = torch.randn(33, 40, device="cuda", requires_grad=True)
        y = layer(x)[0]
        y.square().sum().backward()
        gx, gw = x.grad.clone(), layer.weight.grad.clone()
        gb = None if layer.bias is None else layer.bias.grad.clone()
        run = None if layer.mean_shift is None else layer.mean_shift.running_mean.clone()
        # the same layer on the torch path: float64 on the CPU, distances by the broadcast formula
        ref = NormDist(40, 24, **kw).double()
        ref.load_state_dict({k: v.double().cpu() for k, v in layer.state_dict().items()})
        if ref.mean_shift is not None:
            ref.mean_shift.running_mean.zero_()
        ref.p = 8.0
        import sys
        M = sys.modules["core.modules.norm_dist"]  # (the attribute of that name on the package is the function)
        orig = M.norm_dist
        M.norm_dist = lambda inp, w, pp, groups=1, tag=None: orig(inp, w, pp, groups, use_custom_cuda_func=False)
        try:
            x64 = x.detach().double().cpu().requires_grad_(True)
            y64 = ref(x64)[0]
            y64.square().sum().backward()
        finally:
            M.norm_dist = orig
        assert rel_err(y.detach().cpu().numpy(), y64.detach().numpy()) < 1e-5
        assert rel_err(gx.cpu().numpy(), x64.grad.numpy()) < 1e-4
        assert rel_err(gw.cpu().numpy(), ref.weight.grad.numpy()) < 1e-4
        if gb is not None:
            assert rel_err(gb.cpu().numpy(), ref.bias.grad.numpy()) < 1e-5
        if run is not None:
            assert rel_err(run.cpu().numpy(), ref.mean_shift.running_mean.numpy()) < 1e-5
