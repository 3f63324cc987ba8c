"""GPU parity: finite-p distance forward and backward against the float64 CPU oracle (<= 1e-5 relative)."""
import numpy as np
import pytest

from oracle import norm_dist_oracle as O
from util import make_inputs, assert_close, backward_tolerances, gpu_norm_forward, gpu_norm_backward

pytestmark = pytest.mark.gpu

SHAPES = [(5, 7, 33, 1, 1), (64, 96, 256, 1, 1), (130, 200, 1000, 1, 1), (32, 10, 512, 1, 1), (48, 64, 120, 2, 1),
          (3, 8, 24, 4, 5), (4, 40, 72, 1, 64), (2, 24, 36, 2, 49), (512, 80, 2080, 1, 1), (512, 5120, 104, 1, 1),
          (2048, 2048, 72, 1, 1), (2, 512, 40, 1, 1024), (130, 260, 1000, 1, 1)]
PS = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 9.0, 10.0, 2.5, 9.99, 10.5, 13.7, 100.0, 1000.0]


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("B,CO,CI,G,HW", SHAPES[:3] + SHAPES[4:8])
def test_forward(B, CO, CI, G, HW, p):
    x, w, _ = make_inputs(500 + B, B, CO, CI, G, HW)
    exp = O.norm_dist_forward(x, w, p, G)
    got = gpu_norm_forward(x, w, p, G)
    assert_close(got, exp, what="p=%g" % p)


@pytest.mark.parametrize("p", [8.0, 3.0, 2.5, 13.7])
@pytest.mark.parametrize("shape", SHAPES[8:13])
def test_forward_large_tile_configurations(shape, p):
    # shapes chosen so that the launcher picks the 128 x 80 (k split over wave groups) and 128 x 128 configurations
    B, CO, CI, G, HW = shape
    x, w, _ = make_inputs(501, B, CO, CI, G, HW)
    assert_close(gpu_norm_forward(x, w, p, G), O.norm_dist_forward(x, w, p, G), what="p=%g" % p)


def test_forward_uniform_inputs_config1_like():
    # config-1-like statistics: x uniform[0,1], w N(0, 1/CI)
    r = np.random.RandomState(3)
    B, CO, CI = 96, 160, 3072
    x = r.rand(B, CI, 1).astype(np.float32)
    w = (r.randn(CO, CI) / np.sqrt(CI)).astype(np.float32)
    assert_close(gpu_norm_forward(x, w, 8.0), O.norm_dist_forward(x, w, 8.0), what="p=8 uniform")


def test_forward_floor_and_scale_extremes():
    xz = np.zeros((4, 16, 1), np.float32)
    wz = np.zeros((6, 16), np.float32)
    for p in (2.0, 8.0, 3.5):
        assert_close(gpu_norm_forward(xz, wz, p), O.norm_dist_forward_f32(xz, wz, p), what="all-equal p=%g" % p)
    assert_close(gpu_norm_forward(xz, wz, 13.7), O.norm_dist_forward(xz, wz, 13.7), tol=1e-4, what="all-equal p=13.7")
    # large and small magnitudes must not overflow / underflow the normalised path
    x, w, _ = make_inputs(502, 8, 12, 200)
    for scale in (1e-6, 1e6):
        xs, ws = (x * scale).astype(np.float32), (w * scale).astype(np.float32)
        for p in (13.7, 300.0):
            assert_close(gpu_norm_forward(xs, ws, p), O.norm_dist_forward(xs, ws, p), what="scale %g p=%g" % (scale, p))


@pytest.mark.parametrize("CI", [150, 300])  # tiled kernel / lanes-over-k kernel
@pytest.mark.parametrize("p", [3.0, 8.0, 13.7])
def test_forward_with_max(p, CI):
    x, w, _ = make_inputs(503, 20, 30, CI, 1, 1)
    mx, _ = O.inf_dist_forward(x, w)
    mx = (mx * 1.25).astype(np.float32)  # any normaliser >= the true maximum gives the same value
    exp = O.norm_dist_forward(x, w, p) if p > 10 else None
    got = gpu_norm_forward(x, w, p, max_output=mx)
    # value = m * (sum (|t|/m)^p + (1e-10/m)^p)^(1/p) == ||t||_p up to the negligible phantom term
    d = np.abs(x[:, None, :, 0].astype(np.float64) - w[None].astype(np.float64))
    ref = (d ** p).sum(-1) ** (1 / p)
    assert_close(got[:, :, 0], ref, what="with_max p=%g" % p)
    if exp is not None:
        assert_close(got, exp, what="with_max vs forward p=%g" % p)


@pytest.mark.parametrize("p", [1.0, 1.5, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 2.5, 9.0, 13.7, 100.0])
@pytest.mark.parametrize("B,CO,CI,G,HW", [SHAPES[0], SHAPES[1], SHAPES[4], SHAPES[5], SHAPES[6], SHAPES[7]])
def test_backward(B, CO, CI, G, HW, p):
    x, w, g = make_inputs(600 + B, B, CO, CI, G, HW)
    out = O.norm_dist_forward(x, w, p, G).astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out, p, G)
    assert_close(gx, ex, what="grad_input p=%g" % p)
    assert_close(gw, ew, what="grad_weight p=%g" % p)
    gx2, _ = gpu_norm_backward(g, x, w, out, p, G, with_weight=False)
    assert_close(gx2, ex, what="grad_input (input only) p=%g" % p)


@pytest.mark.parametrize("p", [8.0, 13.7])
@pytest.mark.parametrize("B,CO,CI", [(130, 200, 1000), (600, 70, 130), (32, 10, 512), (65, 40, 200), (128, 33, 70),
                                     (256, 20, 130), (300, 50, 64), (384, 17, 200), (640, 30, 100), (768, 18, 65),
                                     (1100, 20, 70)])
def test_backward_more_shapes(B, CO, CI, p):
    # every workgroup size of the row-split kernel with one and with several row chunks (128-, 256- and 512-row
    # chunks, chosen by padded work), ragged slabs and co chunks, tiny CO
    x, w, g = make_inputs(700 + B, B, CO, CI)
    out = O.norm_dist_forward(x, w, p).astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out, p)
    gx, gw = gpu_norm_backward(g, x, w, out, p)
    assert_close(gx, ex, what="grad_input")
    assert_close(gw, ew, what="grad_weight")


@pytest.mark.parametrize("p", [1.5, 100.0, 200.0])
@pytest.mark.parametrize("B,CO,CI", [(65, 40, 200), (130, 50, 130), (300, 33, 70)])
def test_backward_padded_row_chunks_with_a_second_factor_array(B, CO, CI, p):
    """Waves whose rows are all padding of the last row chunk skip their units; the variants that read a second factor
    array (grad_output apart below p = 2, the compensation term from p = 65 on) must keep both request streams going."""
    x, w, g = make_inputs(900 + B, B, CO, CI)
    out = O.norm_dist_forward(x, w, p).astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out, p)
    gx, gw = gpu_norm_backward(g, x, w, out, p)
    tol_x, tol_w = backward_tolerances(g, x, w, out, p, 1, ex, ew)
    assert_close(gx, ex, tol=tol_x, what="grad_input B=%d p=%g" % (B, p))
    assert_close(gw, ew, tol=tol_w, what="grad_weight B=%d p=%g" % (B, p))


@pytest.mark.parametrize("p", [1.0, 1.5, 8.0, 13.7])
@pytest.mark.parametrize("B,CO,CI,G,HW", [(3, 20, 70, 1, 100), (7, 12, 66, 2, 130)])
def test_backward_conv_layout_many_positions(B, CO, CI, G, HW, p):
    # conv layout with enough positions for the transposed-scratch path: ragged 64 x 64 transpose tiles, several
    # row chunks, groups
    x, w, g = make_inputs(800 + B, B, CO, CI, G, HW)
    out = O.norm_dist_forward(x, w, p, G).astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out, p, G)
    assert_close(gx, ex, what="grad_input p=%g" % p)
    assert_close(gw, ew, what="grad_weight p=%g" % p)


@pytest.mark.parametrize("p", [16.0, 24.5, 48.0, 100.0, 1000.0])
@pytest.mark.parametrize("dist", ["normal", "uniform", "one_outlier", "unit_weights"])
def test_forward_large_p_probe_and_skipping(dist, p):
    # large enough (2.7e8 pairs) for the device-side probe: normal data with small weights (the pairs that count line
    # up over the columns) selects the pair-skipping operator, uniform data (many pairs near the maximum) and, at
    # moderate p, unit-variance weights (pairs that count spread over all of a wave's steps) the plain one;
    # "one_outlier" puts a single huge pair late in every row, so the running maximum jumps after most of the row was
    # accumulated against a much smaller one
    B, CO, CI = 256, 512, 2048
    r = np.random.RandomState(17)
    if dist == "uniform":
        x = r.rand(B, CI, 1).astype(np.float32)
    else:
        x = r.randn(B, CI, 1).astype(np.float32)
    w = (r.randn(CO, CI) / (1.0 if dist == "unit_weights" else np.sqrt(CI))).astype(np.float32)
    if dist == "one_outlier":
        x[:, 1900, 0] += 40.0
    got = gpu_norm_forward(x, w, p)
    rows = [0, 3, 100, 255]
    assert_close(got[rows], O.norm_dist_forward(x[rows], w, p), what="%s p=%g" % (dist, p))
    # never below the maximum, never above K^(1/p) times it
    mx = O.inf_dist_forward(x[rows], w)[0]
    assert np.all(got[rows] >= mx * (1 - 1e-6)) and np.all(got[rows] <= mx * CI ** (1.0 / p) * (1 + 1e-6))


@pytest.mark.parametrize("p", [17.0, 30.0, 48.0, 100.0, 1000.0])
@pytest.mark.parametrize("dist", ["normal", "uniform"])
def test_backward_large_p_probe_and_skipping(dist, p):
    # the backward's twin of the probe test: normal data runs the term-skipping kernel, uniform data the plain one
    B, CO, CI = 256, 512, 2048
    r = np.random.RandomState(23)
    x = (r.rand(B, CI, 1) if dist == "uniform" else r.randn(B, CI, 1)).astype(np.float32)
    w = (r.randn(CO, CI) / np.sqrt(CI)).astype(np.float32)
    g = r.randn(B, CO, 1).astype(np.float32)
    g[5] *= 1e-3  # rows with small grad_output must keep their (small) gradients
    out = gpu_norm_forward(x, w, p)
    gx, gw = gpu_norm_backward(g, x, w, out, p)
    rows, cols = [0, 5, 100, 255], slice(100, 132)
    # conditioning: the fp32 rounding of |t| / out (6e-8 relative) is raised to the power p - 1 with the term, so no
    # fp32 evaluation agrees with the float64 oracle to better than about 1e-7 * p on the large elements: the
    # tolerance is 1e-5, or twice the error of a plain float32 evaluation of the same terms where that misses 1e-5
    ex, _ = O.norm_dist_backward(g[rows], x[rows], w, out[rows], p, with_weight=False)
    tol, _ = backward_tolerances(g[rows], x[rows], w, out[rows], p, 1, ex, None, skipping=True)
    assert_close(gx[rows], ex, tol=tol, what="grad_input rows %s p=%g" % (dist, p))
    # (one row: the comparison rests on a few elements, so the bound is that of the four rows together)
    assert_close(gx[5:6], ex[1:2], tol=2 * tol, what="grad_input of the row with small grad_output")
    _, ew = O.norm_dist_backward(g[:, cols], x, w[cols], out[:, cols], p)
    _, tol = backward_tolerances(g[:, cols], x, w[cols], out[:, cols], p, 1, None, ew, skipping=True)
    assert_close(gw[cols], ew, tol=tol, what="grad_weight columns %s p=%g" % (dist, p))


GROUP_SHAPES = [(16, 24, 1024, 2, 1),    # lanes-over-k forward and co-split backward, two groups
                (600, 128, 1024, 2, 1),  # k range split over workgroups, two groups; row-split backward, two chunks
                (40, 36, 1536, 3, 1)]    # three groups, 512 inputs each


@pytest.mark.parametrize("p", [3.0, 8.0, 13.7, 100.0])
@pytest.mark.parametrize("B,CO,CI,G,HW", GROUP_SHAPES)
def test_groups_on_every_kernel_family(B, CO, CI, G, HW, p):
    x, w, g = make_inputs(900 + B, B, CO, CI, G, HW)
    out = O.norm_dist_forward(x, w, p, G)
    assert_close(gpu_norm_forward(x, w, p, G), out, what="forward p=%g" % p)
    out32 = out.astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out32, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out32, p, G)
    tol_x, tol_w = backward_tolerances(g, x, w, out32, p, G, ex, ew)  # 1e-5 unless plain float32 cannot reach it
    assert_close(gx, ex, tol=tol_x, what="grad_input p=%g" % p)
    assert_close(gw, ew, tol=tol_w, what="grad_weight p=%g" % p)


@pytest.mark.parametrize("p", [2.0, 8.0, 13.7, 100.0])
@pytest.mark.parametrize("B,CO,CI,G,HW", [(1, 16, 1152, 1, 64), (2, 40, 1200, 2, 49), (1, 8, 2048, 1, 20)])
def test_conv_layout_with_k_split_over_workgroups(B, CO, CI, G, HW, p):
    x, w, g = make_inputs(990 + HW, B, CO, CI, G, HW)
    out = O.norm_dist_forward(x, w, p, G)
    assert_close(gpu_norm_forward(x, w, p, G), out, what="forward p=%g" % p)
    out32 = out.astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out32, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out32, p, G)
    tol_x, tol_w = backward_tolerances(g, x, w, out32, p, G, ex, ew)  # 1e-5 unless plain float32 cannot reach it
    assert_close(gx, ex, tol=tol_x, what="grad_input p=%g" % p)
    assert_close(gw, ew, tol=tol_w, what="grad_weight p=%g" % p)


def test_large_p_probe_in_the_conv_layout():
    # the probe, the pair-skipping forward and the term-skipping backward on hw-contiguous inputs (2.4e8 pairs);
    # the backward also goes through the transposed scratch copies
    B, CO, CI, HW, p = 8, 64, 1152, 400, 100.0
    x, w, g = make_inputs(1001, B, CO, CI, 1, HW)
    out = gpu_norm_forward(x, w, p)
    assert_close(out[:2], O.norm_dist_forward(x[:2], w, p), what="forward")
    gx, gw = gpu_norm_backward(g, x, w, out, p)
    ex, _ = O.norm_dist_backward(g[:2], x[:2], w, out[:2], p, with_weight=False)
    tol, _ = backward_tolerances(g[:2], x[:2], w, out[:2], p, 1, ex, None)
    assert_close(gx[:2], ex, tol=tol, what="grad_input")
    _, ew = O.norm_dist_backward(g[:, :4], x, w[:4], out[:, :4], p)
    _, tol = backward_tolerances(g[:, :4], x, w[:4], out[:, :4], p, 1, None, ew)
    assert_close(gw[:4], ew, tol=tol, what="grad_weight")


@pytest.mark.parametrize("p", [1.0, 1.5, 2.0, 3.0, 5.0, 8.0, 9.0, 13.7, 100.0])
@pytest.mark.parametrize("B", [1, 3, 8, 9, 16, 17, 32])
def test_backward_row_chunks_of_small_batches(B, p):
    # the small-batch backward works on chunks of 8, 16 or 32 rows (reference: the same kernels for every batch size,
    # core/cuda/norm_dist_cuda.cu:590-623): every exponent family at batch sizes on and next to the chunk borders,
    # both entry points, two groups, ragged co and ci
    CO, CI, G = 52, 330, 2
    x, w, g = make_inputs(1200 + B, B, CO, CI, G, 1)
    out = gpu_norm_forward(x, w, p, G)
    ex, ew = O.norm_dist_backward(g, x, w, out, p, G)
    gx, gw = gpu_norm_backward(g, x, w, out, p, G)
    tol_x, tol_w = backward_tolerances(g, x, w, out, p, G, ex, ew)
    assert_close(gx, ex, tol=tol_x, what="grad_input B=%d p=%g" % (B, p))
    assert_close(gw, ew, tol=tol_w, what="grad_weight B=%d p=%g" % (B, p))
    gx2, _ = gpu_norm_backward(g, x, w, out, p, G, with_weight=False)
    assert_close(gx2, ex, tol=tol_x, what="input-only entry point B=%d p=%g" % (B, p))
