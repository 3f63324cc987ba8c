"""The large-p kernels come in variants (plain, pair skipping, and for the backward skipping by bounds) of which
device-side probes normally choose one, and only on large problems.  ndist_set_skip_mode forces a variant, also on
small problems, so that each of them is checked against the oracle on shapes the oracle finishes quickly: ragged
tiles, groups, the conv layout, a k range split over workgroups, extreme input scales, data with one dominant pair
per output (identity-initialised layers) and data where almost every pair counts."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import assert_close, backward_tolerances, gpu_inf_forward, gpu_norm_forward, gpu_norm_backward

pytestmark = pytest.mark.gpu

MODES = [(1, 0), (1, 1), (0, -1)]  # (skip, bounds): term-by-term skipping, skipping by bounds, plain
SHAPES = [  # B, CO, CI, G, HW
    (37, 50, 333, 1, 1),       # ragged everything
    (600, 128, 1024, 2, 1),    # two groups; backward in five 128-row chunks (4-wave workgroups)
    (520, 96, 640, 1, 1),      # 520 rows: 128-row chunks again, last one nearly empty
    (512, 64, 512, 1, 1),      # backward: one 512-row chunk (16-wave workgroups)
    (1000, 40, 320, 1, 1),     # backward: two 512-row chunks, grad_weight summed by atomics
    (250, 48, 640, 1, 1),      # backward: one 256-row chunk (8-wave workgroups)
    (3, 24, 200, 1, 49),       # conv layout, odd number of positions
    (2, 40, 1200, 2, 64),      # conv layout, vector paths, k range split over workgroups
]


@pytest.fixture
def skip_mode():
    from core import _C
    yield _C.set_skip_mode
    _C.set_skip_mode(-1, -1)


def _data(kind, B, CO, CI, G, HW, seed):
    r = np.random.RandomState(seed)
    x = r.randn(B, CI, HW).astype(np.float32)
    w = r.randn(CO, CI // G).astype(np.float32)
    if kind == "diagonal":       # one dominant pair per output, like the identity initialisation of the layers
        w *= 0.3
        for n in range(CO):
            w[n, n % (CI // G)] = -10.0
    elif kind == "small_w":      # the pairs that count line up over the outputs
        w /= np.sqrt(CI // G)
    elif kind == "uniform":      # almost every pair counts
        x = r.rand(B, CI, HW).astype(np.float32)
        w = r.rand(CO, CI // G).astype(np.float32)
    g = r.randn(B, CO, HW).astype(np.float32)
    return x, w, g


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("kind", ["diagonal", "small_w", "uniform"])
@pytest.mark.parametrize("p", [16.0, 37.5, 200.0])
@pytest.mark.parametrize("B,CO,CI,G,HW", SHAPES)
def test_forced_variants_match_the_oracle(skip_mode, B, CO, CI, G, HW, p, kind, mode):
    skip_mode(*mode)
    x, w, g = _data(kind, B, CO, CI, G, HW, seed=B + CI)
    out = gpu_norm_forward(x, w, p, G)
    assert_close(out, O.norm_dist_forward(x, w, p, G), what="forward %s p=%g mode=%s" % (kind, p, mode))
    ex, ew = O.norm_dist_backward(g, x, w, out, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out, p, G)
    tol_x, tol_w = backward_tolerances(g, x, w, out, p, G, ex, ew, skipping=mode[0] != 0)
    assert_close(gx, ex, tol=tol_x, what="grad_input %s p=%g mode=%s" % (kind, p, mode))
    assert_close(gw, ew, tol=tol_w, what="grad_weight %s p=%g mode=%s" % (kind, p, mode))


@pytest.mark.parametrize("mode", MODES[:2])
@pytest.mark.parametrize("scale", [1e-6, 1e6])
def test_forced_variants_at_extreme_scales(skip_mode, scale, mode):
    skip_mode(*mode)
    B, CO, CI = 300, 64, 512
    x, w, g = _data("diagonal", B, CO, CI, 1, 1, seed=5)
    x, w = (x * scale).astype(np.float32), (w * scale).astype(np.float32)
    p = 64.0
    out = gpu_norm_forward(x, w, p)
    assert_close(out, O.norm_dist_forward(x, w, p), what="forward scale %g" % scale)
    ex, ew = O.norm_dist_backward(g, x, w, out, p)
    gx, gw = gpu_norm_backward(g, x, w, out, p)
    tol_x, tol_w = backward_tolerances(g, x, w, out, p, 1, ex, ew, skipping=mode[0] != 0)
    assert_close(gx, ex, tol=tol_x, what="grad_input scale %g" % scale)
    assert_close(gw, ew, tol=tol_w, what="grad_weight scale %g" % scale)


def test_mode_is_reset():
    # the fixture restores the probes; a forward on a small problem then takes the plain path again (same result)
    from core import _C
    _C.set_skip_mode(-1, -1)
    x, w, _ = _data("small_w", 20, 30, 100, 1, 1, seed=1)
    a = gpu_norm_forward(x, w, 50.0)
    _C.set_skip_mode(1, 1)
    b = gpu_norm_forward(x, w, 50.0)
    _C.set_skip_mode(-1, -1)
    assert_close(a, b, what="plain against skipping")


def _inf_data(kind, B, CO, CI, G, seed):
    if kind == "ties":  # few distinct values: many pairs attain the maximum, the lowest k must win
        r = np.random.RandomState(seed)
        x = r.randint(-3, 4, size=(B, CI, 1)).astype(np.float32) * 0.5
        w = r.randint(-3, 4, size=(CO, CI // G)).astype(np.float32) * 0.25
        return x, w
    if kind == "zeros":  # nothing exceeds the 1e-10 floor
        return np.zeros((B, CI, 1), np.float32), np.zeros((CO, CI // G), np.float32)
    x, w, _ = _data(kind, B, CO, CI, G, 1, seed)
    return x, w


@pytest.mark.parametrize("skip", [1, 0])
@pytest.mark.parametrize("kind", ["diagonal", "small_w", "uniform", "ties", "zeros"])
@pytest.mark.parametrize("B,CO,CI,G,HW", [s for s in SHAPES if s[4] == 1] + [(300, 400, 700, 1, 1), (130, 330, 1000, 1, 1)])
def test_inf_forward_with_and_without_tile_skipping(skip_mode, B, CO, CI, G, HW, kind, skip):
    """p = inf on the fully-connected layout: forced on, the k-tile skipping operator (seeds and tile bounds) serves
    these small problems too; values and arg-max codes are bit-exact either way."""
    skip_mode(skip, -1)
    x, w = _inf_data(kind, B, CO, CI, G, seed=3 * B + CI)
    ey, epos = O.inf_dist_forward(x, w, G)
    y, pos = gpu_inf_forward(x, w, G)
    assert np.array_equal(y, ey), "%s skip=%d: values differ" % (kind, skip)
    assert np.array_equal(pos, epos), "%s skip=%d: arg-max codes differ" % (kind, skip)
    y2, _ = gpu_inf_forward(x, w, G, with_pos=False)
    assert np.array_equal(y2, ey), "%s skip=%d: values of the no-grad forward differ" % (kind, skip)


@pytest.mark.parametrize("skip", [1, 0])
@pytest.mark.parametrize("eps", [0.0, 0.05, 3.0])
@pytest.mark.parametrize("kind", ["diagonal", "small_w", "uniform", "ties", "zeros"])
@pytest.mark.parametrize("B,CO,CI,G,HW", [(600, 128, 1024, 2, 1), (520, 96, 640, 1, 1), (300, 400, 700, 1, 1),
                                          (130, 330, 1000, 1, 1)])
def test_bound_forward_with_and_without_tile_skipping(skip_mode, B, CO, CI, G, HW, kind, eps, skip):
    """Interval bounds with and without arg-max on the fully-connected layout: forced on, the k-tile skipping
    operator serves these small problems too; bounds and arg-max codes are bit-exact either way."""
    from util import gpu_bound_forward
    skip_mode(skip, -1)
    x, w = _inf_data(kind, B, CO, CI, G, seed=5 * B + CI)
    r = np.random.RandomState(B)
    xl = (x - eps * r.rand(*x.shape)).astype(np.float32)
    xu = (x + eps * r.rand(*x.shape)).astype(np.float32)
    # a few inverted boxes (they collapse to their midpoints) and one box that contains every weight
    xl[1], xu[1] = xu[1].copy(), xl[1].copy()
    xl[2, ::3], xu[2, ::3] = xu[2, ::3].copy(), xl[2, ::3].copy()
    xl[3], xu[3] = -99.0, 99.0
    el, eu, epl, epu = O.bound_inf_dist_forward(xl, xu, w, G)
    yl, yu, _, _ = gpu_bound_forward(xl, xu, w, G, with_pos=False)
    assert np.array_equal(yl, el), "%s eps=%g skip=%d: lower bounds differ" % (kind, eps, skip)
    assert np.array_equal(yu, eu), "%s eps=%g skip=%d: upper bounds differ" % (kind, eps, skip)
    yl, yu, pl, pu = gpu_bound_forward(xl, xu, w, G)
    assert np.array_equal(yl, el) and np.array_equal(yu, eu), "%s eps=%g skip=%d: bounds with arg-max differ" % (kind, eps, skip)
    assert np.array_equal(pl, epl), "%s eps=%g skip=%d: lower arg-max codes differ" % (kind, eps, skip)
    assert np.array_equal(pu, epu), "%s eps=%g skip=%d: upper arg-max codes differ" % (kind, eps, skip)
