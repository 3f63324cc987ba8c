"""The p = inf and interval-bound backwards on layers with 2048 outputs and more per group (the grad_input kernel then
runs 1024 threads per batch row) and with arg-max codes that pile up on one element: activations against small
weights (all outputs of a row name the same input) and weights with one planted entry per row (all batch rows of an
output name the same weight) -- the cases in which lanes are summed before they add.  Ragged sizes on purpose."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import assert_close, gpu_bound_backward, gpu_bound_forward, gpu_inf_backward, gpu_inf_forward

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["small_w", "diagonal", "dense"])
@pytest.mark.parametrize("B,CO,CI,G", [(33, 2050, 515, 1), (70, 4100, 258, 2), (17, 8191, 33, 1)])
def test_wide_layers_with_clustered_codes(B, CO, CI, G, kind):
    r = np.random.RandomState(B + CO)
    x = r.randn(B, CI, 1).astype(np.float32)
    w = r.randn(CO, CI // G).astype(np.float32) * (0.02 if kind == "small_w" else 1.0)
    if kind == "diagonal":
        w[np.arange(CO), np.arange(CO) % (CI // G)] = -10.0
    g, g2 = r.randn(B, CO, 1).astype(np.float32), r.randn(B, CO, 1).astype(np.float32)
    out, pos = gpu_inf_forward(x, w, G)
    eo, ep = O.inf_dist_forward(x, w, G)
    assert np.array_equal(out, eo) and np.array_equal(pos, ep)
    gx, gw = gpu_inf_backward(g, pos, CI, G)
    ex, ew = O.inf_dist_backward(g, ep, CI, G)
    assert_close(gx, ex, what="grad_input")
    assert_close(gw, ew, what="grad_weight")
    yl, yu, pl, pu = gpu_bound_forward(x - 0.1, x + 0.1, w, G)
    oyl, oyu, opl, opu = O.bound_inf_dist_forward(x - 0.1, x + 0.1, w, G)
    assert np.array_equal(yl, oyl) and np.array_equal(yu, oyu) and np.array_equal(pl, opl) and np.array_equal(pu, opu)
    bxl, bxu, bw = gpu_bound_backward(g, g2, pl, pu, CI, G)
    exl, exu, ebw = O.bound_inf_dist_backward(g, g2, opl, opu, CI, G)
    assert_close(bxl, exl, what="grad_inputL")
    assert_close(bxu, exu, what="grad_inputU")
    assert_close(bw, ebw, what="grad_weight (bounds)")
