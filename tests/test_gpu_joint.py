"""The joint entry points (a layer's infinity distance and its interval bounds in one call, pre-pass over the weights
shared): bit for bit what the two separate entry points give, which the oracle pins (reference: the two operator calls
of core/modules/norm_dist.py:30-34)."""
import numpy as np
import pytest
import torch

from oracle import norm_dist_oracle as O

pytestmark = pytest.mark.gpu

SHAPES = [(64, 48, 200, 1, 1), (300, 520, 1030, 1, 1), (96, 64, 256, 2, 1), (3, 10, 36, 1, 50)]


@pytest.mark.parametrize("forced", [False, True])
@pytest.mark.parametrize("B,CO,CI,G,HW", SHAPES)
def test_joint_forward_matches_the_oracle_and_the_separate_calls(B, CO, CI, G, HW, forced):
    from core import _C
    r = np.random.RandomState(B + CI)
    x = r.randn(B, CI, HW).astype(np.float32)
    rad = (r.rand(B, CI, HW) * 0.2).astype(np.float32)
    xl, xu = x - rad, x + rad
    w = (r.randn(CO, CI // G) / np.sqrt(CI // G)).astype(np.float32)
    xd, xld, xud, wd = (torch.from_numpy(a).cuda() for a in (x, xl, xu, w))
    new = lambda dt=torch.float32: torch.empty(B, CO, HW, device="cuda", dtype=dt)
    y, yl, yu, p, pl, pu = new(), new(), new(), new(torch.int32), new(torch.int32), new(torch.int32)
    y2, yl2, yu2 = new(), new(), new()
    if forced:
        _C.set_skip_mode(1, -1)  # the seeded k-tile skipping variants (and with them the shared pre-pass) on small problems
    try:
        _C.inf_and_bound_forward(xd, xld, xud, wd, y, p, yl, yu, pl, pu, G)
        _C.inf_and_bound_forward_nograd(xd, xld, xud, wd, y2, yl2, yu2, G)
    finally:
        _C.set_skip_mode(-1, -1)
    eo, ep = O.inf_dist_forward(x, w, G)
    el, eu, epl, epu = O.bound_inf_dist_forward(xl, xu, w, G)
    for got, exp in ((y, eo), (p, ep), (yl, el), (yu, eu), (pl, epl), (pu, epu), (y2, eo), (yl2, el), (yu2, eu)):
        np.testing.assert_array_equal(got.cpu().numpy(), exp)


def test_layer_certification_path_uses_the_joint_call():
    from core.modules import NormDist
    torch.manual_seed(2)
    layer = NormDist(300, 520, bias=False, mean_shift=True).cuda().eval()
    layer.p = float("inf")
    x = torch.randn(256, 300, device="cuda")
    with torch.no_grad():
        a = layer(x, x - 0.1, x + 0.1)
        # the same through the separate operators
        from core.norm_dist import norm_dist, bound_inf_dist
        y = norm_dist(x.unsqueeze(-1), layer.weight, float("inf"))
        yl, yu = bound_inf_dist((x - 0.1).unsqueeze(-1), (x + 0.1).unsqueeze(-1), layer.weight)
        b = layer._shift_and_bias(y, yl, yu)
    for s, t in zip(a, b):
        assert torch.equal(s, t.squeeze(-1))
    assert bool((a[1] <= a[0]).all()) and bool((a[0] <= a[2]).all())
