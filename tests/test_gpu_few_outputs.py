"""Few outputs over a long reduction (the 10-class last layer; reference: core/cuda/norm_dist_cuda.cu:35-148,
inf_dist_cuda.cu:106-198, bound_inf_dist_cuda.cu:121-238 compute such layers with the same kernels as any other):
the library spreads the k range of such problems over the lanes of a wave and over the four waves of a workgroup,
256 k per wave and step.  Reductions whose length falls on, just behind and between those steps — waves with no step
at all, a last step with a few k, k that are not a multiple of the 16-byte loads — against the oracle: bit-exact for
p = inf and the interval bounds (values and codes), 1e-5 relative for finite p."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import assert_close, gpu_bound_forward, gpu_inf_forward, gpu_norm_forward, make_inputs

pytestmark = pytest.mark.gpu

LENGTHS = [256, 257, 260, 511, 768, 1023, 1024, 1028, 2304, 5120]


@pytest.mark.parametrize("CI", LENGTHS)
@pytest.mark.parametrize("B,CO,G", [(6, 10, 1), (3, 7, 1), (33, 12, 2)])
def test_max_reductions(B, CO, G, CI):
    CI = CI // G * G
    x, w, _ = make_inputs(900 + CI, B, CO, CI, G)
    x[0, CI - 1, 0] = 7.5    # a maximum in the very last k
    w[CO - 1, 0] = -6.5      # and one in the first
    eo, ep = O.inf_dist_forward(x, w, G)
    out, pos = gpu_inf_forward(x, w, G)
    assert np.array_equal(out, eo) and np.array_equal(pos, ep)
    out2, _ = gpu_inf_forward(x, w, G, with_pos=False)
    assert np.array_equal(out2, eo)
    xl, xu = (x - 0.05).astype(np.float32), (x + 0.05).astype(np.float32)
    expect = O.bound_inf_dist_forward(xl, xu, w, G)
    for with_pos in (True, False):
        got = gpu_bound_forward(xl, xu, w, G, with_pos=with_pos)
        for e, v in zip(expect, got):
            assert v is None or np.array_equal(e, v)


@pytest.mark.parametrize("CI", LENGTHS)
@pytest.mark.parametrize("p", [1.0, 3.5, 8.0, 13.7, 100.0])
def test_finite_exponents(p, CI):
    x, w, _ = make_inputs(950 + CI, 6, 10, CI)
    assert_close(gpu_norm_forward(x, w, p), O.norm_dist_forward(x, w, p), what="p=%g CI=%d" % (p, CI))
