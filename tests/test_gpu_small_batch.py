"""Finite-p forward on batches of 8 to 64 rows against wide layers: the shapes for which the launcher picks the
16 x 256, 32 x 128 and 64 x 80 tiles (more outputs than the lanes-over-k kernel takes, fewer rows than a 128-row
tile).  Ragged sizes, groups, integer and general exponents, the one-pass normalised sum and its two-pass fallback."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import assert_close, gpu_norm_backward, gpu_norm_forward, make_inputs

pytestmark = pytest.mark.gpu

SHAPES = [(8, 5120, 1024, 1), (16, 4100, 516, 2), (31, 2051, 700, 1), (32, 4096, 512, 1), (40, 2048, 513, 1),
          (64, 1536, 768, 3)]


@pytest.mark.parametrize("p", [1.0, 3.0, 8.0, 9.3, 13.7, 40.0, 100.0])
@pytest.mark.parametrize("B,CO,CI,G", SHAPES)
def test_forward_small_batch_wide_layer(B, CO, CI, G, p):
    x, w, g = make_inputs(B + CO, B, CO, CI, G)
    out = gpu_norm_forward(x, w, p, G)
    assert_close(out, O.norm_dist_forward(x, w, p, G), what="forward p=%g" % p)


@pytest.mark.parametrize("B,CO,CI,G", SHAPES[:3])
def test_backward_small_batch_wide_layer(B, CO, CI, G):
    x, w, g = make_inputs(B, B, CO, CI, G)
    out = gpu_norm_forward(x, w, 8.0, G)
    gx, gw = gpu_norm_backward(g, x, w, out, 8.0, G)
    ex, ew = O.norm_dist_backward(g, x, w, out, 8.0, G)
    assert_close(gx, ex, what="grad_input")
    assert_close(gw, ew, what="grad_weight")
