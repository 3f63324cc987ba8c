"""p = inf forward through hot k-tiles (reference: core/cuda/inf_dist_cuda.cu:14-198,248-317): on data where a few
k decide every maximum the library computes the outputs from those k-tiles alone.  Values and arg-max codes must be
bit-identical to the oracle whichever side (rows of x, rows of w) selects the tiles, also when the selection is
forced onto data it would not be chosen for (then nearly every tile is hot), with ties, floors, NaN, infinities,
groups and ragged sizes.  ndist_set_skip_mode(1, .) makes the seeded paths serve these small shapes,
ndist_set_hot_mode picks the side."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import gpu_bound_forward, gpu_inf_forward

pytestmark = pytest.mark.gpu

SHAPES = [  # B, CO, CI, G
    (37, 50, 333, 1),      # ragged everything, scalar loads
    (200, 300, 1024, 1),   # full tiles, 16-byte loads
    (130, 96, 1056, 2),    # two groups, a last partial 64-tile word
    (64, 16, 4100, 1),     # more than 128 tiles: masks of five words, partial last tile
    (5, 700, 96, 1),       # few rows, many columns
]


@pytest.fixture
def modes():
    from core import _C
    _C.set_skip_mode(1, -1)
    yield _C.set_hot_mode
    _C.set_hot_mode(-1)
    _C.set_skip_mode(-1, -1)


def _data(kind, B, CO, CI, G, seed):
    r = np.random.RandomState(seed)
    K = CI // G
    x = r.randn(B, CI, 1).astype(np.float32)
    w = r.randn(CO, K).astype(np.float32)
    if kind == "small_w":        # the outliers of x decide
        w /= np.sqrt(K)
    elif kind == "diagonal":     # a planted entry per row of w decides
        w *= 0.3
        for n in range(CO):
            w[n, n % K] = -10.0
    elif kind == "ties":         # small integers: many equal maxima, the lowest k must win
        x = r.randint(-3, 4, size=x.shape).astype(np.float32)
        w = r.randint(-3, 4, size=w.shape).astype(np.float32)
    elif kind == "floor":        # every difference at or below the 1e-10 floor: value 1e-10, code 0
        x = np.repeat(r.randn(1, CI, 1).astype(np.float32), B, axis=0)
        w = np.concatenate([np.tile(x[0, g * K:(g + 1) * K, 0], (CO // G, 1)) for g in range(G)])
        w = np.ascontiguousarray(w, dtype=np.float32)
    elif kind == "special":      # NaN and infinities in both operands
        w /= np.sqrt(K)
        x[1, 5, 0] = np.nan
        x[2, 7 % CI, 0] = np.inf
        x[3, 9 % CI, 0] = -np.inf
        x[3, 10 % CI, 0] = np.inf
        w[2, 3] = np.nan
        w[4 % CO, 11 % K] = np.inf
        w[5 % CO, 7 % K] = np.inf   # inf - inf against x[2]
    return x, w


@pytest.mark.parametrize("mode", [2, 3, 1, -1, 0])
@pytest.mark.parametrize("kind", ["small_w", "diagonal", "normal", "ties", "floor", "special"])
@pytest.mark.parametrize("B,CO,CI,G", SHAPES)
def test_hot_tiles_match_the_oracle(modes, B, CO, CI, G, kind, mode):
    if kind == "floor" and CO % G:
        pytest.skip("needs whole groups")
    modes(mode)
    x, w = _data(kind, B, CO, CI, G, seed=B + CO)
    eo, ep = O.inf_dist_forward(x, w, G)
    out, pos = gpu_inf_forward(x, w, G)
    assert np.array_equal(out.view(np.uint32), eo.view(np.uint32)), "values %s mode %d" % (kind, mode)
    assert np.array_equal(pos, ep), "codes %s mode %d" % (kind, mode)
    out2, _ = gpu_inf_forward(x, w, G, with_pos=False)
    assert np.array_equal(out2.view(np.uint32), eo.view(np.uint32)), "values without codes %s mode %d" % (kind, mode)


def _boxes(kind, x, r):
    """Input bounds around x: narrow boxes, boxes as wide as the data (the lower reduction then sees its floor),
    some inverted boxes (they collapse to their midpoint), and with `special` data the NaN / infinities of x."""
    radius = {"wide": 2.0}.get(kind, 8.0 / 255.0)
    xl, xu = (x - radius).astype(np.float32), (x + radius).astype(np.float32)
    flip = r.rand(*x.shape) < 0.02
    xl[flip], xu[flip] = xu[flip].copy(), xl[flip].copy()
    return xl, xu


@pytest.mark.parametrize("mode", [2, 3, 1, -1, 0])
@pytest.mark.parametrize("kind", ["small_w", "diagonal", "normal", "ties", "floor", "special", "wide"])
@pytest.mark.parametrize("B,CO,CI,G", SHAPES)
def test_hot_tiles_interval_bounds_match_the_oracle(modes, B, CO, CI, G, kind, mode):
    """The same for the interval bounds (reference: core/cuda/bound_inf_dist_cuda.cu:63,148-151,203-213,225-232):
    both bounds and both arg codes, with the "no gradient" code where the lower reduction stays at its floor."""
    if kind == "floor" and CO % G:
        pytest.skip("needs whole groups")
    modes(mode)
    x, w = _data("small_w" if kind == "wide" else kind, B, CO, CI, G, seed=B + CO + 1)
    xl, xu = _boxes(kind, x, np.random.RandomState(B))
    el, eu, epl, epu = O.bound_inf_dist_forward(xl, xu, w, G)
    yl, yu, pl, pu = gpu_bound_forward(xl, xu, w, G)
    what = "%s mode %d" % (kind, mode)
    assert np.array_equal(yl.view(np.uint32), el.view(np.uint32)), "lower bound " + what
    assert np.array_equal(yu.view(np.uint32), eu.view(np.uint32)), "upper bound " + what
    assert np.array_equal(pl, epl), "codes of the lower bound " + what
    assert np.array_equal(pu, epu), "codes of the upper bound " + what
    yl2, yu2, _, _ = gpu_bound_forward(xl, xu, w, G, with_pos=False)
    assert np.array_equal(yl2.view(np.uint32), el.view(np.uint32)), "lower bound without codes " + what
    assert np.array_equal(yu2.view(np.uint32), eu.view(np.uint32)), "upper bound without codes " + what


@pytest.mark.parametrize("mode", [-1, 2, 3])
@pytest.mark.parametrize("kind", ["small_w", "diagonal", "normal"])
@pytest.mark.parametrize("B,CO,CI", [(64, 1024, 1024), (8, 2560, 2560), (150, 800, 1000)])
def test_small_batches_unforced(B, CO, CI, kind, mode):
    """Batches below the size of the k-tile skipping kernels still try the hot tiles first (from 5e7 pairs on), with
    the plain kernels queued behind the decision: no forcing of the seeded paths here."""
    from core import _C
    _C.set_hot_mode(mode)
    try:
        x, w = _data(kind, B, CO, CI, 1, seed=B)
        eo, ep = O.inf_dist_forward(x, w)
        out, pos = gpu_inf_forward(x, w)
        assert np.array_equal(out, eo) and np.array_equal(pos, ep), "%s mode %d" % (kind, mode)
        out2, _ = gpu_inf_forward(x, w, with_pos=False)
        assert np.array_equal(out2, eo), "without codes %s mode %d" % (kind, mode)
        xl, xu = _boxes(kind, x, np.random.RandomState(4))
        expect = O.bound_inf_dist_forward(xl, xu, w)
        for with_pos in (True, False):
            got = gpu_bound_forward(xl, xu, w, with_pos=with_pos)
            for e, v in zip(expect, got):
                assert v is None or np.array_equal(e, v), "interval bounds %s mode %d" % (kind, mode)
    finally:
        _C.set_hot_mode(-1)


def test_decision_follows_the_data(modes):
    """With the counts deciding, both kinds of sparse data and dense data give the oracle's bits at a size where the
    choice matters (the kernel names in a profile tell which path ran; here only the results are checked)."""
    modes(-1)
    B, CO, CI = 256, 1024, 2048
    for kind in ("small_w", "diagonal", "normal"):
        x, w = _data(kind, B, CO, CI, 1, seed=11)
        eo, ep = O.inf_dist_forward(x, w)
        out, pos = gpu_inf_forward(x, w)
        assert np.array_equal(out, eo) and np.array_equal(pos, ep), kind
        xl, xu = _boxes(kind, x, np.random.RandomState(3))
        expect = O.bound_inf_dist_forward(xl, xu, w)
        got = gpu_bound_forward(xl, xu, w)
        for e, v in zip(expect, got):
            assert np.array_equal(e, v), "interval bounds " + kind


@pytest.mark.parametrize("kind", ["normal", "late"])
def test_long_reductions_where_little_can_be_dropped(modes, kind):
    """The k-tile skipping kernels on long reductions where they can drop little: dense data, and `late` data that is
    dense up to three quarters of the k range and has its decisive entries behind that (the thresholds stay loose
    for most of the walk).  Values and codes are the oracle's (hot tiles off, so that the tiled kernels run)."""
    modes(0)
    B, CO, CI = 130, 200, 4096
    x, w = _data("normal", B, CO, CI, 1, seed=21)
    if kind == "late":
        x[:, 3 * CI // 4:, 0] *= 0.05
        w[:, 3 * CI // 4:] *= 0.05
        x[np.arange(B), 3 * CI // 4 + np.arange(B), 0] = 9.0
    eo, ep = O.inf_dist_forward(x, w)
    out, pos = gpu_inf_forward(x, w)
    assert np.array_equal(out, eo) and np.array_equal(pos, ep), kind
    out2, _ = gpu_inf_forward(x, w, with_pos=False)
    assert np.array_equal(out2, eo), "without codes " + kind
    xl, xu = _boxes(kind, x, np.random.RandomState(5))
    expect = O.bound_inf_dist_forward(xl, xu, w)
    for with_pos in (True, False):
        got = gpu_bound_forward(xl, xu, w, with_pos=with_pos)
        for e, v in zip(expect, got):
            assert v is None or np.array_equal(e, v), "interval bounds " + kind


@pytest.mark.parametrize("kind", ["normal", "small_w", "diagonal", "mixed"])
def test_unforced_routes_at_a_size_where_all_three_are_queued(kind):
    """Nothing forced, a problem large enough for the hot-tile plan and both dense kernels behind it: dense data
    (`normal`: every tile hot on both sides, the plain tiled kernel runs), sparse data (the hot tiles run) and
    `mixed` data (a quarter of the rows of x carry outliers: too many hot tiles for the hot-tile kernel, few enough
    for the tile-skipping one) all give the oracle's bits, with and without codes, distance and interval bounds."""
    B, CO, CI = 256, 1024, 2048
    x, w = _data("small_w" if kind == "mixed" else kind, B, CO, CI, 1, seed=31)
    if kind == "mixed":
        r = np.random.RandomState(32)
        x *= 0.05
        rows = np.arange(0, B, 4)
        x[rows] = (r.randn(len(rows), CI, 1) * (r.rand(len(rows), CI, 1) < 0.3) * 4).astype(np.float32)
    eo, ep = O.inf_dist_forward(x, w)
    out, pos = gpu_inf_forward(x, w)
    assert np.array_equal(out, eo) and np.array_equal(pos, ep), kind
    out2, _ = gpu_inf_forward(x, w, with_pos=False)
    assert np.array_equal(out2, eo), "without codes " + kind
    xl, xu = _boxes(kind, x, np.random.RandomState(6))
    expect = O.bound_inf_dist_forward(xl, xu, w)
    for with_pos in (True, False):
        got = gpu_bound_forward(xl, xu, w, with_pos=with_pos)
        for e, v in zip(expect, got):
            assert v is None or np.array_equal(e, v), "interval bounds " + kind
