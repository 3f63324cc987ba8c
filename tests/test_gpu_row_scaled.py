"""The one-pass forward for 10 < p <= 48 (sum normalised by a bound of the maximum that is known before the reduction
starts) against the oracle, forced on for shapes the oracle finishes quickly: ragged tiles, groups, a k range split
over workgroups, extreme input scales, and outputs whose true maximum lies so far below the bound that their sum
underflows and the pass over marked outputs has to recompute them (rows of w that nearly equal rows of x, all-zero
data).  ndist_set_scaled_mode(0) must give the same values within the operator's tolerance."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import assert_close, gpu_norm_forward

pytestmark = pytest.mark.gpu

SHAPES = [  # B, CO, CI, G
    (37, 50, 333, 1),       # ragged everything, scalar loads in the row pass
    (600, 128, 1024, 2),    # two groups
    (512, 80, 640, 1),
    (8, 2048, 2048, 1),     # few rows: k range split over workgroups
    (1000, 40, 320, 1),
]


@pytest.fixture
def scaled_mode():
    from core import _C
    yield _C.set_scaled_mode
    _C.set_scaled_mode(-1)


def _data(B, CO, CI, G, seed, w_scale):
    r = np.random.RandomState(seed)
    x = r.randn(B, CI, 1).astype(np.float32)
    w = (r.randn(CO, CI // G) * w_scale).astype(np.float32)
    return x, w


@pytest.mark.parametrize("w_scale", [0.02, 1.0])
@pytest.mark.parametrize("p", [10.5, 13.7, 25.0, 48.0])
@pytest.mark.parametrize("B,CO,CI,G", SHAPES)
def test_one_pass_matches_the_oracle(scaled_mode, B, CO, CI, G, p, w_scale):
    x, w = _data(B, CO, CI, G, B + CI, w_scale)
    ref = O.norm_dist_forward(x, w, p, G)
    scaled_mode(1)
    assert_close(gpu_norm_forward(x, w, p, G), ref, what="one pass p=%g" % p)
    scaled_mode(0)
    assert_close(gpu_norm_forward(x, w, p, G), ref, what="two passes p=%g" % p)


@pytest.mark.parametrize("p", [13.7, 48.0])
@pytest.mark.parametrize("scale", [1e-6, 1e6])
def test_one_pass_at_extreme_scales(scaled_mode, p, scale):
    x, w = _data(300, 64, 512, 1, 5, 0.3)
    x, w = (x * scale).astype(np.float32), (w * scale).astype(np.float32)
    scaled_mode(1)
    assert_close(gpu_norm_forward(x, w, p), O.norm_dist_forward(x, w, p), what="scale %g" % scale)


@pytest.mark.parametrize("p", [13.7, 48.0])
def test_outputs_far_below_the_bound_are_recomputed(scaled_mode, p):
    """Rows of w that repeat a row of x up to 1e-4: the maxima of those outputs are 1e-4 against a bound of about 8,
    (1e-5)^p is far below the float range.  Every such output, and only those, takes the exact route; each must
    still meet the tolerance on its own."""
    B, CO, CI = 96, 160, 640
    r = np.random.RandomState(11)
    x = r.randn(B, CI, 1).astype(np.float32)
    w = r.randn(CO, CI).astype(np.float32)
    for n in range(0, CO, 3):
        w[n] = x[(7 * n) % B, :, 0] + (1e-4 * r.randn(CI)).astype(np.float32)
    w[5] = x[3, :, 0]  # an exact copy: the distance is the 1e-10 floor's term alone
    ref = O.norm_dist_forward(x, w, p)
    scaled_mode(1)
    out = gpu_norm_forward(x, w, p)
    assert np.all(out >= 0)
    assert np.all(np.abs(out - ref) <= 1e-5 * np.abs(ref)), "an output far below the bound is off"


def test_all_zero_data(scaled_mode):
    x = np.zeros((40, 256, 1), np.float32)
    w = np.zeros((48, 256), np.float32)
    scaled_mode(1)
    out = gpu_norm_forward(x, w, 13.7)
    assert_close(out, O.norm_dist_forward(x, w, 13.7), what="zeros")
