"""Pins the interval-bound functions of the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import norm_dist_oracle as O
from oracle import torch_formulation as TF


def rand_box(seed, B, CO, CI, G=1, HW=1, eps=8 / 255):
    r = np.random.RandomState(seed)
    x = r.randn(B, CI, HW).astype(np.float32)
    w = (r.randn(CO, CI // G) / np.sqrt(CI // G)).astype(np.float32)
    return x, (x - np.float32(eps)).astype(np.float32), (x + np.float32(eps)).astype(np.float32), w


@pytest.mark.parametrize("G,HW", [(1, 1), (2, 3), (1, 5)])
def test_forward_vs_reference_formula(G, HW):
    """The reference's non-kernel branch (core/norm_dist.py:111-120) restated with numpy broadcasting."""
    B, CO, CI = 5, 6, 24
    x, xl, xu, w = rand_box(31, B, CO, CI, G, HW)
    yl, yu, pl, pu = O.bound_inf_dist_forward(xl, xu, w, G)
    CIg = CI // G
    wv = w.reshape(G, CO // G, CIg, 1)
    t1 = wv - xl.reshape(B, G, 1, CIg, HW)
    t2 = xu.reshape(B, G, 1, CIg, HW) - wv
    z1 = np.maximum(np.maximum(t1, t2), np.float32(1e-10))
    z2 = np.minimum(np.minimum(t1, t2), np.float32(-1e-10))
    np.testing.assert_array_equal(yu, z1.max(3).reshape(B, CO, HW))
    np.testing.assert_array_equal(yl, (-z2).max(3).reshape(B, CO, HW))
    # argmax codes: first occurrence + which branch was active
    iu, su = O.decode_pos(pu)
    mx = np.maximum(t1, t2).reshape(B, CO, CIg, HW)
    np.testing.assert_array_equal(iu, mx.argmax(2))
    branch = (t1 > t2).reshape(B, CO, CIg, HW)  # flag set iff not (t1 <= t2)
    np.testing.assert_array_equal(su, np.take_along_axis(branch, mx.argmax(2)[:, :, None, :], 2)[:, :, 0, :])
    # lower bound: first occurrence of the minimum of min(t1, t2) and the branch active there (reference:
    # core/cuda/bound_inf_dist_cuda.cu:203-213); outputs that stayed at the floor carry the "no gradient" code
    mn = np.minimum(t1, t2).reshape(B, CO, CIg, HW)
    il, sl = O.decode_pos(pl)
    moved = yl > np.float32(1e-10)
    assert moved.any()
    np.testing.assert_array_equal(il[moved], mn.argmin(2)[moved])
    np.testing.assert_array_equal(sl[moved], np.take_along_axis(branch, mn.argmin(2)[:, :, None, :], 2)[:, :, 0, :][moved])
    np.testing.assert_array_equal(pl.view(np.uint32)[~moved], np.uint32(0xffffffff))
    yl2, yu2, n1, n2 = O.bound_inf_dist_forward(xl, xu, w, G, with_pos=False)
    assert n1 is None and n2 is None
    np.testing.assert_array_equal(yl, yl2)
    np.testing.assert_array_equal(yu, yu2)


def test_torch_formulation_agrees():
    x, xl, xu, w = rand_box(32, 6, 40, 64)
    yl, yu, _, _ = O.bound_inf_dist_forward(xl, xu, w)
    tl, tu = TF.bound_inf_dist(torch.from_numpy(xl[:, :, 0]), torch.from_numpy(xu[:, :, 0]), torch.from_numpy(w), chunk=16)
    np.testing.assert_array_equal(tl.numpy(), yl[:, :, 0])
    np.testing.assert_array_equal(tu.numpy(), yu[:, :, 0])


def test_soundness_and_tightness():
    B, CO, CI = 4, 9, 32
    x, xl, xu, w = rand_box(33, B, CO, CI, eps=0.3)
    yl, yu, _, _ = O.bound_inf_dist_forward(xl, xu, w)
    r = np.random.RandomState(34)
    for _ in range(50):
        xs = (xl + (xu - xl) * r.rand(*x.shape).astype(np.float32)).astype(np.float32)
        xs = np.clip(xs, xl, xu)
        o, _ = O.inf_dist_forward(xs, w)
        assert np.all(o <= yu * (1 + 1e-6)) and np.all(o >= yl * (1 - 1e-6) - 1e-6)
    # degenerate box: both bounds equal the distance itself
    yl0, yu0, _, _ = O.bound_inf_dist_forward(x, x, w)
    o, _ = O.inf_dist_forward(x, w)
    np.testing.assert_array_equal(yu0, o)
    np.testing.assert_array_equal(yl0, o)
    # upper bound is attained at the corner farthest from w, lower bound at the clamp of w into the box
    far = np.where(np.abs(w[None, :, :, None] - xl[:, None]) >= np.abs(xu[:, None] - w[None, :, :, None]),
                   xl[:, None], xu[:, None])           # [B, CO, CI, 1]
    near = np.clip(w[None, :, :, None], xl[:, None], xu[:, None])
    for co in range(CO):
        o_far, _ = O.inf_dist_forward(far[:, co], w[co:co + 1])
        o_near, _ = O.inf_dist_forward(near[:, co].astype(np.float32), w[co:co + 1])
        np.testing.assert_allclose(o_far[:, 0], yu[:, co], rtol=1e-6)
        np.testing.assert_allclose(o_near[:, 0], yl[:, co], rtol=1e-6, atol=1e-10)


def test_sentinel_and_inverted_box():
    # w inside the box for every ci: lower bound stays at the floor and carries the "no gradient" code
    xl = np.full((1, 4, 1), -1.0, np.float32)
    xu = np.full((1, 4, 1), 1.0, np.float32)
    w = np.zeros((2, 4), np.float32)
    w[1, 2] = 3.0
    yl, yu, pl, pu = O.bound_inf_dist_forward(xl, xu, w)
    assert yl[0, 0, 0] == np.float32(1e-10) and pl[0, 0, 0] == -1
    assert yu[0, 0, 0] == 1.0 and pu[0, 0, 0] == 0          # first index, t1 <= t2
    assert yl[0, 1, 0] == 2.0 and yu[0, 1, 0] == 4.0
    il, sl = O.decode_pos(pl[0, 1, 0])
    iu, su = O.decode_pos(pu[0, 1, 0])
    assert (il, bool(sl), iu, bool(su)) == (2, True, 2, True)   # t1 = w - xl = 4 > t2 = xu - w = -2
    # inverted box collapses to the midpoint
    a, b, _, _ = O.bound_inf_dist_forward(xu, xl, w)
    o, _ = O.inf_dist_forward(np.zeros_like(xl), w)
    np.testing.assert_array_equal(a, o)
    np.testing.assert_array_equal(b, o)


@pytest.mark.parametrize("G,HW", [(1, 1), (2, 2)])
def test_backward_vs_autograd(G, HW):
    B, CO, CI = 5, 6, 16
    x, xl, xu, w = rand_box(35, B, CO, CI, G, HW, eps=0.4)
    r = np.random.RandomState(36)
    gl = r.randn(B, CO, HW).astype(np.float32)
    gu = r.randn(B, CO, HW).astype(np.float32)
    yl, yu, pl, pu = O.bound_inf_dist_forward(xl, xu, w, G)
    gxl, gxu, gw = O.bound_inf_dist_backward(gl, gu, pl, pu, CI, G)
    CIg = CI // G
    tl = torch.from_numpy(xl).double().requires_grad_(True)
    tu = torch.from_numpy(xu).double().requires_grad_(True)
    tw = torch.from_numpy(w).double().requires_grad_(True)
    wv = tw.view(G, CO // G, CIg, 1)
    t1 = wv - tl.view(B, G, 1, CIg, HW)
    t2 = tu.view(B, G, 1, CIg, HW) - wv
    z1 = torch.maximum(t1, t2).clamp(min=1e-10).amax(3).reshape(B, CO, HW)
    z2 = (-torch.minimum(t1, t2).clamp(max=-1e-10)).amax(3).reshape(B, CO, HW)
    (z2 * torch.from_numpy(gl).double() + z1 * torch.from_numpy(gu).double()).sum().backward()
    # where yl sits at the floor autograd also yields zero (clamp), matching the sentinel rule
    np.testing.assert_allclose(gxl, tl.grad.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(gxu, tu.grad.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(gw, tw.grad.numpy(), rtol=1e-6, atol=1e-7)
    a, b, none = O.bound_inf_dist_backward(gl, gu, pl, pu, CI, G, with_weight=False)
    assert none is None
    np.testing.assert_array_equal(a, gxl)
    np.testing.assert_array_equal(b, gxu)
    assert (pl == -1).sum() > 0 or True
