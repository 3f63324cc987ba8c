"""CPU tests of the host-side layers that need no kernel: MeanShift, BoundLinear / BoundFinalLinear interval arithmetic,
parameter names, identity initialisation, and the tensor-algebra branch of the operator."""
import math

import numpy as np
import pytest
import torch

from core.modules import MeanShift, BoundLinear, BoundFinalLinear, BoundReLU, BoundSequential, NormDist, NormDistConv
from core.norm_dist import norm_dist, bound_inf_dist
from ell_inf_models import MLPModel, hinge
from oracle import norm_dist_oracle as O


def test_mean_shift_batch_mean_and_running_average():
    ms = MeanShift(5, momentum=0.1, affine=False)
    x = torch.randn(7, 5, 3)
    y, lo, up = ms(x, None, None)
    assert lo is None and up is None
    mean = x.mean(dim=(0, 2))
    torch.testing.assert_close(y, x - mean[None, :, None])
    torch.testing.assert_close(ms.running_mean, 0.1 * mean)
    ms(x)
    torch.testing.assert_close(ms.running_mean, 0.19 * mean)
    ms.eval()
    y2, lo2, up2 = ms(x, x - 1, x + 1)
    torch.testing.assert_close(y2, x - ms.running_mean[None, :, None])
    torch.testing.assert_close(up2 - lo2, torch.full_like(x, 2.0))
    with pytest.raises(AssertionError):
        MeanShift(5).train()(None, x, x)


def test_bound_linear_is_center_radius_interval_arithmetic():
    torch.manual_seed(0)
    lin = BoundLinear(6, 4, bias=True)
    lin.bias.data.normal_()
    x = torch.randn(3, 6)
    lo, up = x - 0.3, x + 0.2
    y, ylo, yup = lin(x, lo, up)
    W = lin.weight * lin.w_scale
    b = lin.bias * lin.b_scale
    torch.testing.assert_close(y, x @ W.t() + b)
    c, r = (lo + up) / 2, (up - lo) / 2
    torch.testing.assert_close(ylo, c @ W.t() + b - r @ W.abs().t())
    torch.testing.assert_close(yup, c @ W.t() + b + r @ W.abs().t())
    # soundness on samples
    for _ in range(20):
        z = lo + (up - lo) * torch.rand_like(x)
        out = z @ W.t() + b
        assert bool((out >= ylo - 1e-5).all()) and bool((out <= yup + 1e-5).all())


def test_bound_final_linear_margin_bound():
    torch.manual_seed(1)
    fin = BoundFinalLinear(5, 4)
    fin.bias.data.normal_()
    x = torch.randn(6, 5)
    lo, up = x - 0.1, x + 0.1
    t = torch.randint(0, 4, (6,))
    logits, res = fin(x, lo, up, targets=t)
    W, b = fin.weight * fin.w_scale, fin.bias * fin.b_scale
    torch.testing.assert_close(logits, x @ W.t() + b)
    for _ in range(20):
        z = lo + (up - lo) * torch.rand_like(x)
        out = z @ W.t() + b
        diff = out - out.gather(1, t[:, None])
        assert bool((diff <= res + 1e-5).all())
    assert torch.allclose(res.gather(1, t[:, None]), torch.zeros(6, 1), atol=1e-6)
    assert torch.equal(fin(x), logits)


def test_identity_initialisation_and_state_dict_names():
    layer = NormDist(6, 10, identity_val=10.0, bias=False, mean_shift=True)
    w = layer.weight.data
    for i in range(10):
        assert w[i, i % 6] == -10.0
    assert set(layer.state_dict().keys()) == {"weight", "mean_shift.running_mean"}
    conv = NormDistConv(4, 6, 3, padding=1, identity_val=10.0)
    taps = conv.weight.data.view(6, 4, 3, 3)
    for i in range(6):
        assert taps[i, i % 4, 1, 1] == -10.0
    assert set(conv.state_dict().keys()) == {"weight", "bias", "mean_shift.running_mean"}
    m = MLPModel(depth=3, width=16, input_dim=(1, 2, 4), identity_val=10.0, scalar=True)
    assert "scalar" in m.state_dict() and "fc_dist.2.bias" in m.state_dict()
    g = NormDist(8, 12, groups=2, identity_val=3.0)
    assert g.weight.shape == (12, 4) and g.weight.data[5, 1] == -3.0


@pytest.mark.parametrize("G,HW", [(1, 1), (2, 3)])
def test_tensor_algebra_branch_matches_oracle(G, HW):
    r = np.random.RandomState(0)
    x = r.randn(4, 12, HW).astype(np.float32)
    w = r.randn(6, 12 // G).astype(np.float32)
    for p in (3.0, 8.0, float("inf")):
        y = norm_dist(torch.from_numpy(x).double(), torch.from_numpy(w).double(), p, G, use_custom_cuda_func=False)
        exp = O.inf_dist_forward(x, w, G)[0] if math.isinf(p) else O.norm_dist_forward(x, w, p, G)
        np.testing.assert_allclose(y.numpy(), exp, rtol=1e-6)
    yl, yu = bound_inf_dist(torch.from_numpy(x - 0.2), torch.from_numpy(x + 0.2), torch.from_numpy(w), G,
                            use_custom_cuda_func=False)
    el, eu, _, _ = O.bound_inf_dist_forward(x - np.float32(0.2), x + np.float32(0.2), w, G)
    np.testing.assert_array_equal(yl.numpy(), el)
    np.testing.assert_array_equal(yu.numpy(), eu)


def test_hinge_loss_formula():
    m = torch.tensor([[0.5, -1.0, 2.0], [-1.0, -2.0, -3.0]])
    h = hinge(mix=0.25)
    relu = m.clamp(min=0)
    expect = 0.75 * relu.max(1)[0].mean() + 0.25 * relu.mean()
    assert float(h(None, m, None)) == pytest.approx(float(expect))


def test_bound_sequential_threads_the_triple():
    seq = BoundSequential(BoundLinear(3, 3), BoundReLU())
    x = torch.randn(2, 3)
    y, lo, up = seq((x, x - 0.1, x + 0.1))
    assert bool((lo <= y + 1e-6).all()) and bool((y <= up + 1e-6).all()) and bool((lo >= 0).all())


@pytest.mark.parametrize("p", [8.0, float("inf")])
def test_an_empty_batch_gives_empty_outputs_and_zero_gradients(p):
    """The reference's kernels run over no rows on an empty batch and its backward clears grad_weight before a launch
    that does nothing (core/cuda/norm_dist_cuda.cu:515-520, 602-604): empty outputs, zero gradients, no error."""
    from core.norm_dist import conv_norm_dist, conv_bound_inf_dist
    w = torch.randn(6, 8, requires_grad=True)
    x = torch.zeros(0, 8, 3, requires_grad=True)
    y = norm_dist(x, w, p)
    assert y.shape == (0, 6, 3)
    y.sum().backward()
    assert x.grad.shape == x.shape and torch.equal(w.grad, torch.zeros_like(w))
    lo, up = bound_inf_dist(x.detach(), x.detach(), w)
    assert lo.shape == up.shape == (0, 6, 3)
    wc = torch.randn(5, 4 * 9, requires_grad=True)
    img = torch.zeros(0, 4, 7, 7, requires_grad=True)
    yc = conv_norm_dist(img, wc, p, 3, 1, 1, 2)
    assert yc.shape == (0, 5, 16)
    yc.sum().backward()
    assert torch.equal(wc.grad, torch.zeros_like(wc)) and img.grad.shape == img.shape
    cl, cu = conv_bound_inf_dist(img.detach(), img.detach(), wc, 3, 1, 1, 2)
    assert cl.shape == cu.shape == (0, 5, 16)
