"""GPU parity of the fused convolutional entry points (patches extracted inside the kernel) against the CPU oracle on
the patches torch.nn.functional.unfold materialises on the CPU: values bit-exact, as for the unfolded layout.
Reference path: core/modules/norm_dist.py:93-102 (F.unfold, then the operator)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import norm_dist_oracle as O
from util import assert_close

pytestmark = pytest.mark.gpu

CASES = [  # B, C, H, W, CO, G, kernel, dilation, padding, stride
    (2, 3, 8, 8, 5, 1, 3, 1, 1, 1),                # small, OW % 4 == 0: four positions share an output row
    (3, 5, 9, 7, 6, 1, (3, 2), 1, (1, 0), (2, 1)),  # ragged: output width 6, positions cross output rows
    (2, 4, 12, 12, 8, 2, 3, 2, 2, 1),              # dilation, two groups
    (1, 2, 6, 10, 4, 1, (1, 1), 1, 0, 1),          # 1x1 window
    (2, 3, 11, 13, 7, 1, 5, 1, 2, 3),              # stride 3, window 5, output 4 x 5
    (3, 8, 4, 4, 9, 1, 4, 1, 0, 1),                # one output position per image (HW == 1)
    (2, 6, 10, 16, 12, 3, 3, 1, 1, (1, 2)),        # horizontal stride 2 on the shared-row path, three groups
    (4, 16, 32, 32, 128, 1, 3, 1, 1, 1),           # 4096 rows x 128 columns: the large tiles
    (1, 256, 8, 8, 32, 1, 3, 1, 1, 1),             # one output tile, k = 2304: k range split over workgroups
    (2, 40, 16, 16, 200, 1, 3, 1, 1, 1),           # ragged column tiles, k = 360 not a multiple of the stage
    (1, 3, 5, 5, 3, 1, 3, 1, 2, 1),                # padding wider than one tap: whole patches of zeros at corners
    (1, 3, 4, 70, 4, 1, 3, 1, 1, 1),               # wider than one block of 32 pixel columns (the adjoint's halo)
    (1, 2, 5, 75, 3, 1, (2, 5), (1, 2), (0, 3), (1, 2)),  # the same with a wide dilated window and a stride
]


def _case(seed, B, C, H, W, CO, G, k, d, p, s):
    gen = torch.Generator().manual_seed(seed)
    kh, kw = (k, k) if isinstance(k, int) else k
    x = torch.randn(B, C, H, W, generator=gen)
    w = torch.randn(CO, C // G * kh * kw, generator=gen) * 0.5
    return x, w


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", CASES)
def test_conv_inf_dist_forward_nograd(B, C, H, W, CO, G, k, d, p, s):
    from core import _C
    x, w = _case(B * 31 + H, B, C, H, W, CO, G, k, d, p, s)
    patches = F.unfold(x, k, d, p, s)
    expect, _ = O.inf_dist_forward(patches.numpy(), w.numpy(), G)
    out = torch.empty(B, CO, patches.size(2), device="cuda")
    _C.conv_inf_dist_forward_nograd(x.cuda(), w.cuda(), out, G, k, d, p, s)
    np.testing.assert_array_equal(out.cpu().numpy(), expect)
    # and the unfolded path of the library itself
    out2 = torch.empty_like(out)
    _C.inf_dist_forward_nograd(patches.cuda(), w.cuda(), out2, G)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", CASES)
def test_conv_bound_inf_dist_forward_nograd(B, C, H, W, CO, G, k, d, p, s):
    from core import _C
    x, w = _case(B * 37 + W, B, C, H, W, CO, G, k, d, p, s)
    gen = torch.Generator().manual_seed(5)
    radius = torch.rand(x.shape, generator=gen) * 0.3
    lower, upper = x - radius, x + radius
    lower[0, 0, 0, :2], upper[0, 0, 0, :2] = upper[0, 0, 0, :2].clone(), lower[0, 0, 0, :2].clone()  # inverted box
    pl, pu = F.unfold(lower, k, d, p, s), F.unfold(upper, k, d, p, s)
    el, eu, _, _ = O.bound_inf_dist_forward(pl.numpy(), pu.numpy(), w.numpy(), G)
    yl = torch.empty(B, CO, pl.size(2), device="cuda")
    yu = torch.empty_like(yl)
    _C.conv_bound_inf_dist_forward_nograd(lower.cuda(), upper.cuda(), w.cuda(), yl, yu, G, k, d, p, s)
    np.testing.assert_array_equal(yl.cpu().numpy(), el)
    np.testing.assert_array_equal(yu.cpu().numpy(), eu)


TRAIN_CASES = CASES + [
    (1, 2, 150, 150, 3, 1, 3, 1, 1, 1),            # an image plane larger than the scatter kernel's LDS tile: the
                                                   # backward takes the unfolded-gradient + adjoint route
    (2, 64, 8, 8, 16, 1, 3, 1, 1, 1),              # several channel slabs per sample in the image-gradient kernel
    (1, 3, 6, 200, 5, 1, 3, 1, 1, 1),              # rows too long for the second pass on staged image rows: the
                                                   # sorted second pass gathers the patches instead
    (2, 300, 6, 6, 7, 1, 3, 1, 1, 1),              # 300 channels: one workgroup of 1024 threads per compute unit
    (1, 3, 100, 120, 6, 1, 5, 1, 2, 2),            # a larger plane, window 5, stride 2: several row blocks per sample
    (2, 6, 40, 24, 10, 2, (3, 2), (2, 1), (2, 0), (1, 2)),  # dilated rows, strided columns, two groups
]


def _fold(grad_patches, shape, k, d, p, s):
    """adjoint of F.unfold on the CPU (float64 sums, so that the yardstick adds no rounding of its own)"""
    return F.fold(torch.from_numpy(np.asarray(grad_patches, np.float64)), shape[2:], k, d, p, s).numpy()


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", TRAIN_CASES)
def test_conv_inf_dist_forward_codes_and_backward(B, C, H, W, CO, G, k, d, p, s):
    from core import _C
    x, w = _case(B * 41 + C, B, C, H, W, CO, G, k, d, p, s)
    x *= 0.3  # weights dominate: at the image border the winning tap often lies in the padding
    patches = F.unfold(x, k, d, p, s)
    eo, ep = O.inf_dist_forward(patches.numpy(), w.numpy(), G)
    out = torch.empty(B, CO, patches.size(2), device="cuda")
    pos = torch.empty_like(out, dtype=torch.int32)
    _C.conv_inf_dist_forward(x.cuda(), w.cuda(), out, pos, G, k, d, p, s)
    np.testing.assert_array_equal(out.cpu().numpy(), eo)
    np.testing.assert_array_equal(pos.cpu().numpy(), ep)

    g = torch.randn(out.shape, generator=torch.Generator().manual_seed(3))
    ex_patches, ew = O.inf_dist_backward(g.numpy(), ep, patches.size(1), G)
    ex = _fold(ex_patches, x.shape, k, d, p, s)
    gx = torch.full(x.shape, float("nan"), device="cuda")
    gw = torch.full(w.shape, float("nan"), device="cuda")
    _C.conv_inf_dist_backward_input_weight(g.cuda(), pos, gx, gw, G, k, d, p, s)
    assert_close(gx.cpu().numpy(), ex, what="grad_input")
    assert_close(gw.cpu().numpy(), ew, what="grad_weight")
    gx2 = torch.full(x.shape, float("nan"), device="cuda")
    _C.conv_inf_dist_backward_input(g.cuda(), pos, gx2, w.shape, G, k, d, p, s)
    assert_close(gx2.cpu().numpy(), ex, what="grad_input (input only)")


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", TRAIN_CASES)
def test_conv_bound_inf_dist_forward_codes_and_backward(B, C, H, W, CO, G, k, d, p, s):
    from core import _C
    x, w = _case(B * 43 + C, B, C, H, W, CO, G, k, d, p, s)
    x *= 0.3
    radius = torch.rand(x.shape, generator=torch.Generator().manual_seed(6)) * 0.2
    lower, upper = x - radius, x + radius
    pl, pu = F.unfold(lower, k, d, p, s), F.unfold(upper, k, d, p, s)
    el, eu, epl, epu = O.bound_inf_dist_forward(pl.numpy(), pu.numpy(), w.numpy(), G)
    yl = torch.empty(B, CO, pl.size(2), device="cuda")
    yu = torch.empty_like(yl)
    posl = torch.empty_like(yl, dtype=torch.int32)
    posu = torch.empty_like(posl)
    _C.conv_bound_inf_dist_forward(lower.cuda(), upper.cuda(), w.cuda(), yl, yu, posl, posu, G, k, d, p, s)
    np.testing.assert_array_equal(yl.cpu().numpy(), el)
    np.testing.assert_array_equal(yu.cpu().numpy(), eu)
    np.testing.assert_array_equal(posl.cpu().numpy(), epl)
    np.testing.assert_array_equal(posu.cpu().numpy(), epu)

    gen = torch.Generator().manual_seed(4)
    gl, gu = torch.randn(yl.shape, generator=gen), torch.randn(yl.shape, generator=gen)
    exl_p, exu_p, ew = O.bound_inf_dist_backward(gl.numpy(), gu.numpy(), epl, epu, pl.size(1), G)
    exl, exu = _fold(exl_p, x.shape, k, d, p, s), _fold(exu_p, x.shape, k, d, p, s)
    gxl = torch.full(x.shape, float("nan"), device="cuda")
    gxu = torch.full(x.shape, float("nan"), device="cuda")
    gw = torch.full(w.shape, float("nan"), device="cuda")
    _C.conv_bound_inf_dist_backward_input_weight(gl.cuda(), gu.cuda(), posl, posu, gxl, gxu, gw, G, k, d, p, s)
    assert_close(gxl.cpu().numpy(), exl, what="grad_lower")
    assert_close(gxu.cpu().numpy(), exu, what="grad_upper")
    assert_close(gw.cpu().numpy(), ew, what="grad_weight")
    gxl2 = torch.full(x.shape, float("nan"), device="cuda")
    gxu2 = torch.full(x.shape, float("nan"), device="cuda")
    _C.conv_bound_inf_dist_backward_input(gl.cuda(), gu.cuda(), posl, posu, gxl2, gxu2, w.shape, G, k, d, p, s)
    assert_close(gxl2.cpu().numpy(), exl, what="grad_lower (inputs only)")
    assert_close(gxu2.cpu().numpy(), exu, what="grad_upper (inputs only)")


def test_conv_layer_training_path_matches_the_unfolded_formulation():
    # NormDistConv with gradients (fused kernels) against torch's unfold + the operator on the unfolded tensors
    from core.modules import NormDistConv
    from core.norm_dist import norm_dist, bound_inf_dist
    torch.manual_seed(12)
    conv = NormDistConv(6, 10, 3, padding=1, stride=2, groups=2, bias=False, mean_shift=False).cuda()
    conv.p = float("inf")
    x = torch.randn(3, 6, 12, 12, device="cuda", requires_grad=True)
    lower, upper = x - 0.1, x + 0.1
    y, yl, yu = conv(x, lower, upper)
    gen = torch.Generator().manual_seed(1)
    gy, gl, gu = (torch.randn(y.shape, generator=gen).cuda() for _ in range(3))
    (y * gy + yl * gl + yu * gu).sum().backward()
    gx1, gw1 = x.grad.clone(), conv.weight.grad.clone()
    x.grad = None
    conv.weight.grad = None
    unf = lambda t: F.unfold(t, 3, 1, 1, 2)
    y2 = norm_dist(unf(x), conv.weight, float("inf"), 2)
    yl2, yu2 = bound_inf_dist(unf(lower), unf(upper), conv.weight, 2)
    assert torch.equal(y.flatten(2), y2) and torch.equal(yl.flatten(2), yl2) and torch.equal(yu.flatten(2), yu2)
    (y2 * gy.flatten(2) + yl2 * gl.flatten(2) + yu2 * gu.flatten(2)).sum().backward()
    assert_close(gx1.cpu().numpy(), x.grad.cpu().numpy(), what="grad_input")
    assert_close(gw1.cpu().numpy(), conv.weight.grad.cpu().numpy(), what="grad_weight")


def test_conv_layer_eval_uses_the_fused_kernels_and_matches_training_mode_values():
    # NormDistConv under no_grad (fused kernels) against the same layer with gradients enabled (unfold + operator)
    from core.modules import NormDistConv
    torch.manual_seed(11)
    conv = NormDistConv(6, 10, 3, padding=1, groups=2, bias=True, mean_shift=False).cuda()
    conv.p = float("inf")
    x = torch.randn(3, 6, 12, 12, device="cuda")
    lower, upper = x - 0.1, x + 0.1
    y_train, l_train, u_train = conv(x, lower, upper)
    assert y_train.requires_grad
    with torch.no_grad():
        y_eval, l_eval, u_eval = conv(x, lower, upper)
    assert y_eval.shape == (3, 10, 12, 12)
    assert torch.equal(y_eval, y_train.detach())
    assert torch.equal(l_eval, l_train.detach())
    assert torch.equal(u_eval, u_train.detach())
    assert bool((l_eval <= y_eval).all()) and bool((y_eval <= u_eval).all())


def test_conv_entry_points_reject_bad_arguments():
    from core import _C
    x = torch.randn(2, 4, 8, 8, device="cuda")
    w = torch.randn(6, 4 * 9, device="cuda")
    out = torch.empty(2, 6, 64, device="cuda")
    with pytest.raises(RuntimeError):  # weight does not match C / G * kh * kw
        _C.conv_inf_dist_forward_nograd(x, w[:, :35].contiguous(), out, 1, 3, 1, 1, 1)
    with pytest.raises(RuntimeError):  # output shape of another geometry
        _C.conv_inf_dist_forward_nograd(x, w, out, 1, 3, 1, 0, 1)
    with pytest.raises(RuntimeError):  # window larger than the padded image
        _C.conv_inf_dist_forward_nograd(x, torch.randn(6, 4 * 121, device="cuda"), out, 1, 11, 1, 1, 1)


@pytest.mark.parametrize("p", [1.0, 2.0, 3.0, 8.0, 2.5, 13.7, 40.0])
@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p_,s", CASES)
def test_conv_norm_dist_forward_and_backward(B, C, H, W, CO, G, k, d, p_, s, p):
    """Finite p on images (reference: F.unfold + norm_dist::forward / backward_input_weight,
    core/modules/norm_dist.py:93-102, core/cuda/norm_dist.h:4-17): output and both gradients within 1e-5 of the
    float64 oracle on the patches torch materialises on the CPU, the input gradient folded back by the adjoint of
    unfold."""
    from core import _C
    from util import backward_tolerances
    x, w = _case(B * 41 + H, B, C, H, W, CO, G, k, d, p_, s)
    patches = F.unfold(x, k, d, p_, s)
    expect = O.norm_dist_forward(patches.numpy(), w.numpy(), p, G)
    xd, wd = x.cuda(), w.cuda()
    out = torch.empty(B, CO, patches.size(2), device="cuda")
    _C.conv_norm_dist_forward(xd, wd, out, G, p, k, d, p_, s)
    assert_close(out.cpu().numpy(), expect, what="conv forward p=%g" % p)
    gen = torch.Generator().manual_seed(9)
    g = torch.randn(out.shape, generator=gen)
    ex, ew = O.norm_dist_backward(g.numpy(), patches.numpy(), w.numpy(), out.cpu().numpy(), p, G)
    ex_img = F.fold(torch.from_numpy(ex), (H, W), k, d, p_, s).numpy()
    tol_x, tol_w = backward_tolerances(g.numpy(), patches.numpy(), w.numpy(), out.cpu().numpy(), p, G, ex, ew)
    gx = torch.full_like(xd, float("nan"))
    gw = torch.full_like(wd, float("nan"))
    _C.conv_norm_dist_backward_input_weight(g.cuda(), xd, wd, out, gx, gw, G, p, k, d, p_, s)
    assert_close(gx.cpu().numpy(), ex_img, tol=tol_x, what="conv grad_input p=%g" % p)
    assert_close(gw.cpu().numpy(), ew, tol=tol_w, what="conv grad_weight p=%g" % p)
    gx2 = torch.full_like(xd, float("nan"))
    _C.conv_norm_dist_backward_input(g.cuda(), xd, wd, out, gx2, G, p, k, d, p_, s)
    assert_close(gx2.cpu().numpy(), ex_img, tol=tol_x, what="conv grad_input alone p=%g" % p)


def test_conv_norm_dist_layer_matches_the_unfolded_path():
    """NormDistConv at finite p runs on the image; its output and gradients agree with the same layer fed through
    the library's own unfold + norm_dist (the path it took before)."""
    from core.modules import NormDistConv
    from core.norm_dist import norm_dist, unfold
    torch.manual_seed(3)
    layer = NormDistConv(8, 16, 3, padding=1, p=8.0, bias=False, mean_shift=False).cuda()
    x = torch.randn(4, 8, 12, 12, device="cuda", requires_grad=True)
    y, _, _ = layer(x)
    y.square().sum().backward()
    gx, gw = x.grad.clone(), layer.weight.grad.clone()
    x.grad = None
    layer.weight.grad = None
    y2 = norm_dist(unfold(x, 3, 1, 1, 1), layer.weight, 8.0, 1).view_as(y)
    y2.square().sum().backward()
    assert_close(y.detach().cpu().numpy(), y2.detach().cpu().numpy(), what="layer output")
    assert_close(gx.cpu().numpy(), x.grad.cpu().numpy(), what="layer grad_input")
    assert_close(gw.cpu().numpy(), layer.weight.grad.cpu().numpy(), what="layer grad_weight")


@pytest.mark.parametrize("G,stride", [(1, 1), (2, 2)])
@pytest.mark.parametrize("p", [3.0, 13.7])
def test_conv_norm_dist_backward_in_parts_of_the_batch(p, G, stride, monkeypatch):
    """Large batches run the finite-p backward on images in parts of whole samples, so that the two patch-sized
    scratch buffers stay bounded, grad_weight accumulating over the parts.  With the budget forced down to 0.5 MiB
    per buffer (twice that where the kernel gathers the patches itself, as here; 590 KB of patches per sample at
    stride 1, 147 KB at stride 2) a 9-sample batch takes nine parts, or two of five and four samples: same gradients
    as in one piece, within 1e-5 of the oracle; also with groups."""
    from core import _C
    from util import backward_tolerances
    B, C, H, W, CO, k = 9, 16, 32, 32, 10, 3
    gen = torch.Generator().manual_seed(77)
    x = torch.randn(B, C, H, W, generator=gen)
    w = torch.randn(CO, C // G * k * k, generator=gen) / (C * k * k) ** 0.5
    patches = F.unfold(x, k, 1, 1, stride)
    xd, wd = x.cuda(), w.cuda()
    out = torch.empty(B, CO, patches.size(2), device="cuda")
    _C.conv_norm_dist_forward(xd, wd, out, G, p, k, 1, 1, stride)
    g = torch.randn(out.shape, generator=gen)
    ex, ew = O.norm_dist_backward(g.numpy(), patches.numpy(), w.numpy(), out.cpu().numpy(), p, G)
    ex_img = F.fold(torch.from_numpy(ex), (H, W), k, 1, 1, stride).numpy()
    tol_x, tol_w = backward_tolerances(g.numpy(), patches.numpy(), w.numpy(), out.cpu().numpy(), p, G, ex, ew)
    whole = [torch.full_like(xd, float("nan")), torch.full_like(wd, float("nan"))]
    _C.conv_norm_dist_backward_input_weight(g.cuda(), xd, wd, out, whole[0], whole[1], G, p, k, 1, 1, stride)
    monkeypatch.setenv("NORM_DIST_CONV_PART_MB", "0.5")
    parts = [torch.full_like(xd, float("nan")), torch.full_like(wd, float("nan"))]
    _C.conv_norm_dist_backward_input_weight(g.cuda(), xd, wd, out, parts[0], parts[1], G, p, k, 1, 1, stride)
    for got in (whole, parts):
        assert_close(got[0].cpu().numpy(), ex_img, tol=tol_x, what="grad_input p=%g" % p)
        assert_close(got[1].cpu().numpy(), ew, tol=tol_w, what="grad_weight p=%g" % p)
    only_x = torch.full_like(xd, float("nan"))
    _C.conv_norm_dist_backward_input(g.cuda(), xd, wd, out, only_x, G, p, k, 1, 1, stride)
    assert_close(only_x.cpu().numpy(), ex_img, tol=tol_x, what="input-only entry point in parts p=%g" % p)


@pytest.mark.parametrize("p", [2.0, 8.0])
@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p_,s", [CASES[1], CASES[2], CASES[4], CASES[7], CASES[-1]])
def test_conv_norm_dist_backward_from_patch_rows(B, C, H, W, CO, G, k, d, p_, s, p, monkeypatch):
    """The finite-p backward on images gathers the patches inside its main kernel; NORM_DIST_BWD_GATHER=0 makes it
    write them out as rows first (the route of the term-skipping variants and of batches of at most 32 positions):
    the same rows, so the same gradients bit for bit, and within 1e-5 of the oracle."""
    from core import _C
    from util import backward_tolerances
    x, w = _case(B * 59 + W, B, C, H, W, CO, G, k, d, p_, s)
    patches = F.unfold(x, k, d, p_, s)
    xd, wd = x.cuda(), w.cuda()
    out = torch.empty(B, CO, patches.size(2), device="cuda")
    _C.conv_norm_dist_forward(xd, wd, out, G, p, k, d, p_, s)
    g = torch.randn(out.shape, generator=torch.Generator().manual_seed(5))
    ex, ew = O.norm_dist_backward(g.numpy(), patches.numpy(), w.numpy(), out.cpu().numpy(), p, G)
    ex_img = F.fold(torch.from_numpy(ex), (H, W), k, d, p_, s).numpy()
    tol_x, tol_w = backward_tolerances(g.numpy(), patches.numpy(), w.numpy(), out.cpu().numpy(), p, G, ex, ew)
    got = []
    for mode in ("1", "0"):
        monkeypatch.setenv("NORM_DIST_BWD_GATHER", mode)
        gx, gw = torch.full_like(xd, float("nan")), torch.full_like(wd, float("nan"))
        _C.conv_norm_dist_backward_input_weight(g.cuda(), xd, wd, out, gx, gw, G, p, k, d, p_, s)
        assert_close(gx.cpu().numpy(), ex_img, tol=tol_x, what="grad_input, gather %s" % mode)
        assert_close(gw.cpu().numpy(), ew, tol=tol_w, what="grad_weight, gather %s" % mode)
        got.append((gx.cpu().numpy(), gw.cpu().numpy()))
    np.testing.assert_array_equal(got[0][0], got[1][0])


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", [CASES[2], CASES[6], CASES[7], CASES[9]])
def test_conv_codes_with_the_sorted_second_pass(B, C, H, W, CO, G, k, d, p, s, monkeypatch):
    """The arg-max codes of the image entry points come from one of two second passes (staged image rows where they
    fit LDS, else the sorted gather of patches); NORM_DIST_RESCAN_IMAGE=0 keeps the second one, which must give the
    same bits."""
    from core import _C
    monkeypatch.setenv("NORM_DIST_RESCAN_IMAGE", "0")
    x, w = _case(B * 47 + C, B, C, H, W, CO, G, k, d, p, s)
    patches = F.unfold(x, k, d, p, s)
    eo, ep = O.inf_dist_forward(patches.numpy(), w.numpy(), G)
    out = torch.empty(B, CO, patches.size(2), device="cuda")
    pos = torch.empty_like(out, dtype=torch.int32)
    _C.conv_inf_dist_forward(x.cuda(), w.cuda(), out, pos, G, k, d, p, s)
    np.testing.assert_array_equal(out.cpu().numpy(), eo)
    np.testing.assert_array_equal(pos.cpu().numpy(), ep)
    radius = torch.rand(x.shape, generator=torch.Generator().manual_seed(8)) * 0.2
    lower, upper = x - radius, x + radius
    pl, pu = F.unfold(lower, k, d, p, s), F.unfold(upper, k, d, p, s)
    el, eu, epl, epu = O.bound_inf_dist_forward(pl.numpy(), pu.numpy(), w.numpy(), G)
    yl = torch.empty(B, CO, pl.size(2), device="cuda")
    yu = torch.empty_like(yl)
    posl = torch.empty_like(yl, dtype=torch.int32)
    posu = torch.empty_like(posl)
    _C.conv_bound_inf_dist_forward(lower.cuda(), upper.cuda(), w.cuda(), yl, yu, posl, posu, G, k, d, p, s)
    np.testing.assert_array_equal(posl.cpu().numpy(), epl)
    np.testing.assert_array_equal(posu.cpu().numpy(), epu)


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", [CASES[2], CASES[6], CASES[7]])
def test_conv_grad_weight_sums_in_doubles(B, C, H, W, CO, G, k, d, p, s, monkeypatch):
    """grad_weight of the scatter backward on images is summed in LDS in double precision (nine times the rate of
    float adds on this part) and rounded once; NORM_DIST_SCATTER_F64=0 keeps float adds.  Both within 1e-5 of the
    oracle, for the distance and for the interval bounds, also on gradients spread over 60 binary orders of
    magnitude; infinities and NaNs reach the same weights on both routes."""
    from core import _C
    x, w = _case(B * 61 + C, B, C, H, W, CO, G, k, d, p, s)
    patches = F.unfold(x, k, d, p, s)
    _, ep = O.inf_dist_forward(patches.numpy(), w.numpy(), G)
    lo, up = x - 0.1, x + 0.1
    _, _, epl, epu = O.bound_inf_dist_forward(F.unfold(lo, k, d, p, s).numpy(), F.unfold(up, k, d, p, s).numpy(), w.numpy(), G)
    pos, posl, posu = (torch.from_numpy(a.astype(np.int32)).cuda() for a in (ep, epl, epu))
    gen = torch.Generator().manual_seed(11)
    g = torch.randn(ep.shape, generator=gen)
    g2 = torch.randn(ep.shape, generator=gen)
    wide = g * torch.exp2(torch.randint(-40, 20, g.shape, generator=gen).float())
    bad = g.clone()
    bad[0, 0, 0] = float("inf")
    bad[-1, -1, -1] = float("nan")
    results = {}
    for mode in ("1", "0"):
        monkeypatch.setenv("NORM_DIST_SCATTER_F64", mode)
        for name, grad in (("plain", g), ("wide", wide), ("bad", bad)):
            gx, gw = torch.full_like(x.cuda(), float("nan")), torch.full_like(w.cuda(), float("nan"))
            _C.conv_inf_dist_backward_input_weight(grad.cuda(), pos, gx, gw, G, k, d, p, s)
            results[mode, name] = gw.cpu().numpy()
        gxl, gxu = torch.full_like(x.cuda(), float("nan")), torch.full_like(x.cuda(), float("nan"))
        gwb = torch.full_like(w.cuda(), float("nan"))
        _C.conv_bound_inf_dist_backward_input_weight(g.cuda(), g2.cuda(), posl, posu, gxl, gxu, gwb, G, k, d, p, s)
        results[mode, "bounds"] = gwb.cpu().numpy()
    for name, grad in (("plain", g), ("wide", wide)):
        _, ew = O.inf_dist_backward(grad.numpy(), ep, patches.size(1), G)
        for mode in ("1", "0"):
            assert_close(results[mode, name], ew, what="grad_weight %s, doubles %s" % (name, mode))
    _, _, ewb = O.bound_inf_dist_backward(g.numpy(), g2.numpy(), epl, epu, patches.size(1), G)
    for mode in ("1", "0"):
        assert_close(results[mode, "bounds"], ewb, what="grad_weight of the bounds, doubles %s" % mode)
    a, b = results["1", "bad"], results["0", "bad"]
    assert np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(np.isinf(a), np.isinf(b))
    assert np.isnan(a).any() and np.isinf(a).any()
    fin = np.isfinite(a)
    assert_close(a[fin], b[fin], what="finite weights beside the non-finite ones")


@pytest.mark.parametrize("B,C,H,W,CO,G,k,d,p,s", [CASES[2], CASES[6], CASES[7], TRAIN_CASES[-1], TRAIN_CASES[len(CASES)]])
def test_conv_backward_by_channel_slabs(B, C, H, W, CO, G, k, d, p, s, monkeypatch):
    """The image gradient of the scatter backward comes from one of two kernels (blocks of output rows where the image
    rows under a block fit LDS, else slabs of channels); NORM_DIST_SCATTER_ROWBLOCKS=0 keeps the second one: same
    gradients within 1e-5 of the oracle, for the distance and for the interval bounds.  The 150 x 150 image fits no
    slab: with the row kernels switched off its gradient goes through the unfolded gradient and the adjoint of the
    patch extraction."""
    from core import _C
    x, w = _case(B * 53 + C, B, C, H, W, CO, G, k, d, p, s)
    x *= 0.3
    radius = torch.rand(x.shape, generator=torch.Generator().manual_seed(9)) * 0.2
    lower, upper = x - radius, x + radius
    patches, pl, pu = F.unfold(x, k, d, p, s), F.unfold(lower, k, d, p, s), F.unfold(upper, k, d, p, s)
    _, ep = O.inf_dist_forward(patches.numpy(), w.numpy(), G)
    _, _, epl, epu = O.bound_inf_dist_forward(pl.numpy(), pu.numpy(), w.numpy(), G)
    gen = torch.Generator().manual_seed(10)
    g, gl, gu = (torch.randn(ep.shape, generator=gen) for _ in range(3))
    ex_p, ew = O.inf_dist_backward(g.numpy(), ep, patches.size(1), G)
    exl_p, exu_p, ewb = O.bound_inf_dist_backward(gl.numpy(), gu.numpy(), epl, epu, pl.size(1), G)
    ex, exl, exu = (_fold(t, x.shape, k, d, p, s) for t in (ex_p, exl_p, exu_p))
    pos, posl, posu = (torch.from_numpy(t).cuda() for t in (ep, epl, epu))
    for mode in ("2", "1", "0"):  # blocks of image rows (the default where they fit), of output rows, channel slabs
        monkeypatch.setenv("NORM_DIST_SCATTER_ROWBLOCKS", mode)
        gx = torch.full(x.shape, float("nan"), device="cuda")
        gw = torch.full(w.shape, float("nan"), device="cuda")
        _C.conv_inf_dist_backward_input_weight(g.cuda(), pos, gx, gw, G, k, d, p, s)
        assert_close(gx.cpu().numpy(), ex, what="grad_input, row blocks " + mode)
        assert_close(gw.cpu().numpy(), ew, what="grad_weight, row blocks " + mode)
        gxl = torch.full(x.shape, float("nan"), device="cuda")
        gxu = torch.full(x.shape, float("nan"), device="cuda")
        _C.conv_bound_inf_dist_backward_input_weight(gl.cuda(), gu.cuda(), posl, posu, gxl, gxu, gw, G, k, d, p, s)
        assert_close(gxl.cpu().numpy(), exl, what="grad_lower, row blocks " + mode)
        assert_close(gxu.cpu().numpy(), exu, what="grad_upper, row blocks " + mode)
        assert_close(gw.cpu().numpy(), ewb, what="grad_weight (bounds), row blocks " + mode)
