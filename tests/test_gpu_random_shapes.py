"""GPU parity on a fixed, seeded sample of irregular shapes: every entry point against the oracle.  The shapes are
drawn once (seeded) from ranges that cross the thresholds between kernel families (lanes-over-k / tiled / split k,
row-split / co-split backward, row / tile scatter, thread-per-output / sorted second pass)."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import (make_inputs, assert_close, gpu_inf_forward, gpu_inf_backward, gpu_bound_forward, gpu_bound_backward,
                  gpu_norm_forward, gpu_norm_backward, backward_tolerances)

pytestmark = pytest.mark.gpu


def _shapes():
    r = np.random.RandomState(20240607)
    out = []
    for _ in range(28):
        G = int(r.choice([1, 1, 1, 2, 3]))
        HW = int(r.choice([1, 1, 1, 1, 5, 16, 37, 64]))
        B = int(r.choice([1, 2, 7, 33, 65, 130, 300]))
        CO = G * int(r.choice([1, 3, 10, 40, 70, 130]))
        CI = G * int(r.choice([3, 31, 64, 257, 520, 1100]))
        if B * HW * CO * CI > 6e8:  # keep the oracle fast
            B = max(1, B // 8)
        out.append((B, CO, CI, G, HW))
    return out


SHAPES = _shapes()


@pytest.mark.parametrize("B,CO,CI,G,HW", SHAPES)
def test_inf_and_bounds(B, CO, CI, G, HW):
    x, w, g = make_inputs(B * 7 + CO, B, CO, CI, G, HW)
    eo, ep = O.inf_dist_forward(x, w, G)
    go, gp = gpu_inf_forward(x, w, G)
    np.testing.assert_array_equal(go, eo)
    np.testing.assert_array_equal(gp, ep)
    np.testing.assert_array_equal(gpu_inf_forward(x, w, G, with_pos=False)[0], eo)
    ex, ew = O.inf_dist_backward(g, ep, CI, G)
    gx, gw = gpu_inf_backward(g, ep, CI, G)
    assert_close(gx, ex, what="inf grad_input")
    assert_close(gw, ew, what="inf grad_weight")
    xl, xu = (x - np.float32(0.3)).astype(np.float32), (x + np.float32(0.3)).astype(np.float32)
    el, eu, epl, epu = O.bound_inf_dist_forward(xl, xu, w, G)
    gl, gu, gpl, gpu_ = gpu_bound_forward(xl, xu, w, G)
    for a, b in ((gl, el), (gu, eu), (gpl, epl), (gpu_, epu)):
        np.testing.assert_array_equal(a, b)
    g2 = np.random.RandomState(B).randn(*g.shape).astype(np.float32)
    bl, bu, bw = O.bound_inf_dist_backward(g, g2, epl, epu, CI, G)
    cl, cu, cw = gpu_bound_backward(g, g2, epl, epu, CI, G)
    assert_close(cl, bl, what="bound grad_lower")
    assert_close(cu, bu, what="bound grad_upper")
    assert_close(cw, bw, what="bound grad_weight")


@pytest.mark.parametrize("p", [1.0, 3.0, 8.0, 9.0, 2.5, 13.7, 60.0])
@pytest.mark.parametrize("B,CO,CI,G,HW", SHAPES[::2])
def test_finite_p(B, CO, CI, G, HW, p):
    x, w, g = make_inputs(B * 11 + CI, B, CO, CI, G, HW)
    out = O.norm_dist_forward(x, w, p, G)
    assert_close(gpu_norm_forward(x, w, p, G), out, what="forward p=%g" % p)
    out32 = out.astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out32, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out32, p, G)
    tol_x, tol_w = backward_tolerances(g, x, w, out32, p, G, ex, ew)  # 1e-5 unless plain float32 cannot reach it
    assert_close(gx, ex, tol=tol_x, what="grad_input p=%g" % p)
    assert_close(gw, ew, tol=tol_w, what="grad_weight p=%g" % p)
