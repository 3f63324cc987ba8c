"""GPU parity at the full benchmark shape (B = 512, CI = CO = 5120).  The max-reductions (p = inf forward, interval
bounds; integer-exact work) are compared with the oracle over EVERY output, values and arg-max codes, with the
data-dependent k-tile skipping on (the default at this size) and forced off.  For finite p the oracle evaluates 64 of
the 512 batch rows (rows are independent in the forward and in grad_input) and 640 of the 5120 output features of
grad_weight (features are independent there); size-independent properties cover the rest."""
import numpy as np
import pytest
import torch

from oracle import norm_dist_oracle as O
from util import assert_close, backward_tolerances, rel_err

pytestmark = pytest.mark.gpu

B, CI, CO = 512, 5120, 5120
# 64 rows: the first and last of every 128-row tile and of every 32-row wave strip of the backward, plus a spread
ROWS = sorted(set([0, 1, 31, 32, 127, 128, 255, 256, 300, 383, 384, 448, 510, 511] + list(range(5, 512, 10))))[:64]
COLS = slice(2240, 2880)                      # 640 output features: eight 80-wide tiles, forty 16-co units


@pytest.fixture(scope="module")
def data():
    gen = torch.Generator().manual_seed(2021)
    x = torch.randn(B, CI, 1, generator=gen)
    w = torch.randn(CO, CI, generator=gen) / np.sqrt(CI)
    g = torch.randn(B, CO, 1, generator=gen)
    return x, w, g


@pytest.fixture(scope="module")
def inf_oracle(data):
    x, w, _ = data
    return O.inf_dist_forward(x.numpy(), w.numpy())  # all 512 x 5120 outputs: values and codes


@pytest.mark.parametrize("skip", [-1, 0])  # k-tile skipping as the library chooses (on at this size) / forced off
def test_inf_forward_backward(data, inf_oracle, skip):
    from core import _C
    x, w, g = data
    xd, wd, gd = x.cuda(), w.cuda(), g.cuda()
    eo, ep = inf_oracle
    out = torch.empty(B, CO, 1, device="cuda")
    pos = torch.empty(B, CO, 1, device="cuda", dtype=torch.int32)
    out2 = torch.empty_like(out)
    _C.set_skip_mode(skip, -1)
    try:
        _C.inf_dist_forward(xd, wd, out, pos, 1)
        _C.inf_dist_forward_nograd(xd, wd, out2, 1)
    finally:
        _C.set_skip_mode(-1, -1)
    np.testing.assert_array_equal(out.cpu().numpy(), eo)
    np.testing.assert_array_equal(pos.cpu().numpy(), ep)
    np.testing.assert_array_equal(out2.cpu().numpy(), eo)
    gx = torch.empty_like(xd)
    gw = torch.empty_like(wd)
    _C.inf_dist_backward_input_weight(gd, pos, gx, gw, 1)
    ex, ew = O.inf_dist_backward(g.numpy(), ep, CI)
    assert_close(gx.cpu().numpy(), ex, what="grad_input")
    assert_close(gw.cpu().numpy(), ew, what="grad_weight")
    # conservation: every output moves +-g to one input and the opposite to one weight
    assert abs(float(gx.double().sum() + gw.double().sum())) < 1e-2


@pytest.mark.parametrize("p", [8.0, 13.7, 100.0])  # 100: the probe picks the pair-skipping forward on this data
def test_norm_forward_backward(data, p):
    from core import _C
    x, w, g = data
    xd, wd, gd = x.cuda(), w.cuda(), g.cuda()
    out = torch.empty(B, CO, 1, device="cuda")
    _C.norm_dist_forward(xd, wd, out, 1, p)
    outc = out.cpu().numpy()
    assert_close(outc[ROWS], O.norm_dist_forward(x.numpy()[ROWS], w.numpy(), p), what="forward rows")
    gx = torch.empty_like(xd)
    gw = torch.empty_like(wd)
    _C.norm_dist_backward_input_weight(gd, xd, wd, out, gx, gw, 1, p)
    # grad_input of a row depends on that row only
    ex, _ = O.norm_dist_backward(g.numpy()[ROWS], x.numpy()[ROWS], w.numpy(), outc[ROWS], p, with_weight=False)
    assert_close(gx.cpu().numpy()[ROWS], ex, what="grad_input rows")
    # grad_weight of an output feature depends on that feature only
    _, ew = O.norm_dist_backward(g.numpy()[:, COLS], x.numpy(), w.numpy()[COLS], outc[:, COLS], p)
    assert_close(gw.cpu().numpy()[COLS], ew, what="grad_weight rows")
    # run-to-run: the forward sums in a fixed order, and so does grad_weight while the batch is one row chunk
    # (grad_input is accumulated with float atomics and only repeats to rounding)
    out_again, gw_again, gx_again = torch.empty_like(out), torch.empty_like(gw), torch.empty_like(gx)
    _C.norm_dist_forward(xd, wd, out_again, 1, p)
    assert torch.equal(out, out_again)
    if p < 16:  # from p = 16 on a probe picks the variant, and the skipping ones drop terms in a data-dependent order
        _C.norm_dist_backward_input_weight(gd, xd, wd, out, gx_again, gw_again, 1, p)
        assert torch.equal(gw, gw_again)
        assert rel_err(gx_again.cpu().numpy(), gx.cpu().numpy()) < 1e-6
    # input-only entry point gives the same grad_input
    gx2 = torch.empty_like(xd)
    _C.norm_dist_backward_input(gd, xd, wd, out, gx2, 1, p)
    assert rel_err(gx2.cpu().numpy(), gx.cpu().numpy()) < 1e-5
    # Euler identity over the whole batch: sum_ci dout/dx * (x - w) = out, i.e. with grad_out = 1 ...
    ones = torch.ones_like(gd)
    _C.norm_dist_backward_input_weight(ones, xd, wd, out, gx, gw, 1, p)
    lhs = (gx.double().squeeze(-1) * xd.double().squeeze(-1)).sum() + (gw.double() * wd.double()).sum()
    assert abs(float(lhs) / float(out.double().sum()) - 1.0) < 1e-5


@pytest.mark.parametrize("skip", [-1, 0])
def test_bound_forward(data, skip):
    from core import _C
    x, w, g = data
    xl, xu = (x - 8 / 255), (x + 8 / 255)
    xld, xud, wd = xl.cuda(), xu.cuda(), w.cuda()
    yl = torch.empty(B, CO, 1, device="cuda")
    yu = torch.empty_like(yl)
    pl = torch.empty(B, CO, 1, device="cuda", dtype=torch.int32)
    pu = torch.empty_like(pl)
    yl2 = torch.empty_like(yl)
    yu2 = torch.empty_like(yl)
    _C.set_skip_mode(skip, -1)
    try:
        _C.bound_inf_dist_forward(xld, xud, wd, yl, yu, pl, pu, 1)
        _C.bound_inf_dist_forward_nograd(xld, xud, wd, yl2, yu2, 1)
    finally:
        _C.set_skip_mode(-1, -1)
    el, eu, epl, epu = O.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy())  # every output
    np.testing.assert_array_equal(yl.cpu().numpy(), el)
    np.testing.assert_array_equal(yu.cpu().numpy(), eu)
    np.testing.assert_array_equal(pl.cpu().numpy(), epl)
    np.testing.assert_array_equal(pu.cpu().numpy(), epu)
    np.testing.assert_array_equal(yl2.cpu().numpy(), el)
    np.testing.assert_array_equal(yu2.cpu().numpy(), eu)
    # the box contains x: bounds bracket the distance itself
    out = torch.empty_like(yl)
    _C.inf_dist_forward_nograd(x.cuda(), wd, out, 1)
    assert bool((yl <= out).all()) and bool((out <= yu).all())
    if skip == 0:
        return
    # backward of the bounds at full size, against the oracle's scatter from the oracle's own codes
    gl, gu = g.cuda(), g.flip(0).contiguous().cuda()
    gxl, gxu, gw = torch.empty_like(xld), torch.empty_like(xld), torch.empty_like(wd)
    _C.bound_inf_dist_backward_input_weight(gl, gu, pl, pu, gxl, gxu, gw, 1)
    exl, exu, ew = O.bound_inf_dist_backward(g.numpy(), g.flip(0).contiguous().numpy(), epl, epu, CI)
    assert_close(gxl.cpu().numpy(), exl, what="grad_lower")
    assert_close(gxu.cpu().numpy(), exu, what="grad_upper")
    assert_close(gw.cpu().numpy(), ew, what="grad_weight")


def test_identity_initialised_layer_every_output():
    """The shape the training and certification figures are quoted on: a 5120 x 5120 layer as the reference
    initialises it (unit-variance weights with -10 planted on the diagonal, core/modules/norm_dist.py:18, 47-50),
    batch 512, activations as a mean shift leaves them.  The library's default path there selects the hot k-tiles by
    the rows of w.  Every output and code of the distance, of the interval bounds, of the joint calls and of the
    calls with the weights' pre-pass kept is compared with the oracle (reference: core/cuda/inf_dist_cuda.cu:173-177,
    bound_inf_dist_cuda.cu:203-213)."""
    from core import _C
    gen = torch.Generator().manual_seed(2021)
    x = torch.randn(B, CI, 1, generator=gen) * 1.1
    x -= x.mean(dim=0, keepdim=True)
    w = torch.randn(CO, CI, generator=gen)
    w[torch.arange(CO), torch.arange(CO) % CI] = -10.0
    xl, xu = x - 8 / 255, x + 8 / 255
    eo, ep = O.inf_dist_forward(x.numpy(), w.numpy())
    el, eu, epl, epu = O.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy())
    xd, xld, xud, wd = x.cuda(), xl.cuda(), xu.cuda(), w.cuda()
    new_f = lambda: torch.full((B, CO, 1), float("nan"), device="cuda")
    new_i = lambda: torch.full((B, CO, 1), -7, device="cuda", dtype=torch.int32)
    same = lambda t, e, what: np.testing.assert_array_equal(t.cpu().numpy(), e, err_msg=what)
    out, pos = new_f(), new_i()
    _C.inf_dist_forward(xd, wd, out, pos, 1)
    same(out, eo, "distance"), same(pos, ep, "distance codes")
    out = new_f()
    _C.inf_dist_forward_nograd(xd, wd, out, 1)
    same(out, eo, "distance, no codes")
    yl, yu, pl, pu = new_f(), new_f(), new_i(), new_i()
    _C.bound_inf_dist_forward(xld, xud, wd, yl, yu, pl, pu, 1)
    same(yl, el, "lower"), same(yu, eu, "upper"), same(pl, epl, "lower codes"), same(pu, epu, "upper codes")
    yl, yu = new_f(), new_f()
    _C.bound_inf_dist_forward_nograd(xld, xud, wd, yl, yu, 1)
    same(yl, el, "lower, no codes"), same(yu, eu, "upper, no codes")
    out, pos, yl, yu, pl, pu = new_f(), new_i(), new_f(), new_f(), new_i(), new_i()
    _C.inf_and_bound_forward(xd, xld, xud, wd, out, pos, yl, yu, pl, pu, 1)
    same(out, eo, "joint distance"), same(pos, ep, "joint distance codes")
    same(yl, el, "joint lower"), same(yu, eu, "joint upper")
    same(pl, epl, "joint lower codes"), same(pu, epu, "joint upper codes")
    out, yl, yu = new_f(), new_f(), new_f()
    _C.inf_and_bound_forward_nograd(xd, xld, xud, wd, out, yl, yu, 1)
    same(out, eo, "joint distance, no codes"), same(yl, el, "joint lower, no codes"), same(yu, eu, "joint upper, no codes")
    cache = _C.weight_cache(wd, 1)
    out = new_f()
    _C.inf_dist_forward_nograd_cached(xd, wd, cache, out, 1)
    same(out, eo, "distance, kept pre-pass")
    out, yl, yu = new_f(), new_f(), new_f()
    _C.inf_and_bound_forward_nograd_cached(xd, xld, xud, wd, cache, out, yl, yu, 1)
    same(out, eo, "joint distance, kept pre-pass"), same(yl, el, "joint lower, kept pre-pass")
    same(yu, eu, "joint upper, kept pre-pass")
    # the hot-tile selection forced onto the rows of x (not chosen on this data: nearly every tile is hot there)
    _C.set_hot_mode(2)
    try:
        out, pos = new_f(), new_i()
        _C.inf_dist_forward(xd, wd, out, pos, 1)
    finally:
        _C.set_hot_mode(-1)
    same(out, eo, "distance, x side forced"), same(pos, ep, "distance codes, x side forced")


def test_config1_forward_p8_uniform_inputs():
    # forward only, p = 8: x uniform[0, 1) [512, 3072], w N(0, 1/3072) [5120, 3072]
    from core import _C
    gen = torch.Generator().manual_seed(2021)
    x = torch.rand(512, 3072, 1, generator=gen)
    w = torch.randn(5120, 3072, generator=gen) / np.sqrt(3072)
    out = torch.empty(512, 5120, 1, device="cuda")
    _C.norm_dist_forward(x.cuda(), w.cuda(), out, 1, 8.0)
    assert_close(out.cpu().numpy()[ROWS], O.norm_dist_forward(x.numpy()[ROWS], w.numpy(), 8.0), what="config 1 rows")


def test_conv_shape_inf_and_bounds():
    # the conv benchmark: input [128, 128, 32, 32], 3x3, pad 1 -> unfolded x [128, 1152, 1024], w [128, 1152];
    # the oracle evaluates three of the 128 samples (samples are independent in the forward and in grad_input)
    from core import _C
    from core.norm_dist import unfold
    gen = torch.Generator().manual_seed(2021)
    img = torch.randn(128, 128, 32, 32, generator=gen)
    w = torch.randn(128, 1152, generator=gen) / np.sqrt(1152)
    g = torch.randn(128, 128, 1024, generator=gen)
    SAMPLES = [0, 77, 127]
    xu = unfold(img.cuda(), 3, 1, 1, 1)
    ref_unf = torch.nn.functional.unfold(img[SAMPLES], 3, 1, 1, 1)
    assert torch.equal(xu[SAMPLES].cpu(), ref_unf)
    wd, gd = w.cuda(), g.cuda()
    out = torch.empty(128, 128, 1024, device="cuda")
    pos = torch.empty(128, 128, 1024, device="cuda", dtype=torch.int32)
    _C.inf_dist_forward(xu, wd, out, pos, 1)
    eo, ep = O.inf_dist_forward(ref_unf.numpy(), w.numpy())
    np.testing.assert_array_equal(out[SAMPLES].cpu().numpy(), eo)
    np.testing.assert_array_equal(pos[SAMPLES].cpu().numpy(), ep)
    out2 = torch.empty_like(out)
    _C.inf_dist_forward_nograd(xu, wd, out2, 1)
    assert torch.equal(out, out2)
    gx = torch.empty_like(xu)
    gw = torch.empty_like(wd)
    _C.inf_dist_backward_input_weight(gd, pos, gx, gw, 1)
    ex, _ = O.inf_dist_backward(g.numpy()[SAMPLES], ep, 1152)
    assert_close(gx[SAMPLES].cpu().numpy(), ex, what="conv grad_input")
    # grad_weight needs every sample: conservation against grad_input instead (each output moves +-g to one input
    # and the opposite to one weight), plus the per-co totals
    assert abs(float(gx.double().sum() + gw.double().sum())) < 2e-2
    sign = torch.where(pos < 0, -1.0, 1.0).double()
    per_co = -(gd.double() * sign).sum(dim=(0, 2))
    assert float((gw.double().sum(dim=1) - per_co).abs().max()) < 1e-2
    del gx, out2
    xl, xh = xu - 8 / 255, xu + 8 / 255
    yl = torch.empty_like(out)
    yu = torch.empty_like(out)
    pl = torch.empty_like(pos)
    pu = torch.empty_like(pos)
    _C.bound_inf_dist_forward(xl, xh, wd, yl, yu, pl, pu, 1)
    rl, rh = (ref_unf.cuda() - 8 / 255).cpu().numpy(), (ref_unf.cuda() + 8 / 255).cpu().numpy()
    el, eu, epl, epu = O.bound_inf_dist_forward(rl, rh, w.numpy())
    np.testing.assert_array_equal(yl[SAMPLES].cpu().numpy(), el)
    np.testing.assert_array_equal(yu[SAMPLES].cpu().numpy(), eu)
    np.testing.assert_array_equal(pl[SAMPLES].cpu().numpy(), epl)
    np.testing.assert_array_equal(pu[SAMPLES].cpu().numpy(), epu)
    assert bool((yl <= out).all()) and bool((out <= yu).all())


def _scatter_weight_gradient(g, pos, CO, CI, skip_code=None):
    """grad_weight of a max-reduction from its codes, restated with numpy.bincount: every output (b, co, hw) adds
    -v to weight[co, idx] with idx the low 31 bits of its code and v = +g / -g by the sign bit (reference:
    core/cuda/inf_dist_cuda.cu:237-242); outputs whose code is `skip_code` send nothing."""
    pos = pos.astype(np.int64) & 0xffffffff
    idx = pos & 0x7fffffff
    v = np.where(pos >> 31 == 0, g, -g).astype(np.float64)
    if skip_code is not None:
        v = np.where(pos == skip_code, 0.0, v)
        idx = np.where(pos == skip_code, 0, idx)
    co = np.arange(CO, dtype=np.int64)[None, :, None]
    flat = (co * CI + idx).ravel()
    return -np.bincount(flat, weights=v.ravel(), minlength=CO * CI).reshape(CO, CI)


def test_conv_shape_fused_entry_points():
    # The same conv benchmark through the entry points NormDistConv really calls: images in, patches extracted inside
    # the kernels, image gradients out.  Oracle: F.unfold patches of three samples (values, codes, grad_input of those
    # samples through the adjoint of unfold); grad_weight over all samples from the library's codes by the scatter
    # rule restated in numpy (the codes themselves are pinned by the three samples and by equality with the unfolded
    # path on every sample).
    from core import _C
    import torch.nn.functional as F
    gen = torch.Generator().manual_seed(2021)
    img = torch.randn(128, 128, 32, 32, generator=gen)
    w = torch.randn(128, 1152, generator=gen) / np.sqrt(1152)
    g = torch.randn(128, 128, 1024, generator=gen)
    g2 = torch.randn(128, 128, 1024, generator=gen)
    SAMPLES = [0, 77, 127]
    geo = (1, 3, 1, 1, 1)  # groups, kernel, dilation, padding, stride
    imd, wd, gd, g2d = img.cuda(), w.cuda(), g.cuda(), g2.cuda()
    patches = F.unfold(img[SAMPLES], 3, 1, 1, 1)
    out = torch.empty(128, 128, 1024, device="cuda")
    pos = torch.empty(128, 128, 1024, device="cuda", dtype=torch.int32)
    _C.conv_inf_dist_forward(imd, wd, out, pos, *geo)
    eo, ep = O.inf_dist_forward(patches.numpy(), w.numpy())
    np.testing.assert_array_equal(out[SAMPLES].cpu().numpy(), eo)
    np.testing.assert_array_equal(pos[SAMPLES].cpu().numpy(), ep)
    out_ng = torch.empty_like(out)
    _C.conv_inf_dist_forward_nograd(imd, wd, out_ng, *geo)
    assert torch.equal(out, out_ng)
    # every sample: the unfolded path of the library gives the same values and codes
    from core.norm_dist import unfold
    xu = unfold(imd, 3, 1, 1, 1)
    out_u, pos_u = torch.empty_like(out), torch.empty_like(pos)
    _C.inf_dist_forward(xu, wd, out_u, pos_u, 1)
    assert torch.equal(out, out_u) and torch.equal(pos, pos_u)
    del xu, out_u, pos_u, out_ng
    gx = torch.full_like(imd, float("nan"))
    gw = torch.full_like(wd, float("nan"))
    _C.conv_inf_dist_backward_input_weight(gd, pos, gx, gw, *geo)
    ex_p, _ = O.inf_dist_backward(g.numpy()[SAMPLES], ep, 1152)
    ex = F.fold(torch.from_numpy(ex_p.astype(np.float64)), (32, 32), 3, 1, 1, 1).numpy()
    assert_close(gx[SAMPLES].cpu().numpy(), ex, what="fused conv grad_input")
    assert_close(gw.cpu().numpy(), _scatter_weight_gradient(g.numpy(), pos.cpu().numpy(), 128, 1152),
                 what="fused conv grad_weight")
    gx_only = torch.full_like(imd, float("nan"))
    _C.conv_inf_dist_backward_input(gd, pos, gx_only, w.shape, *geo)
    assert_close(gx_only.cpu().numpy(), gx.cpu().numpy(), what="input-only entry point")  # LDS atomics: no fixed order
    del gx, gx_only
    # interval bounds on the images, eps = 8 / 255
    lo, up = imd - 8 / 255, imd + 8 / 255
    yl, yu = torch.empty_like(out), torch.empty_like(out)
    pl, pu = torch.empty_like(pos), torch.empty_like(pos)
    _C.conv_bound_inf_dist_forward(lo, up, wd, yl, yu, pl, pu, *geo)
    pl_cpu, pu_cpu = F.unfold(lo[SAMPLES].cpu(), 3, 1, 1, 1), F.unfold(up[SAMPLES].cpu(), 3, 1, 1, 1)
    el, eu, epl, epu = O.bound_inf_dist_forward(pl_cpu.numpy(), pu_cpu.numpy(), w.numpy())
    np.testing.assert_array_equal(yl[SAMPLES].cpu().numpy(), el)
    np.testing.assert_array_equal(yu[SAMPLES].cpu().numpy(), eu)
    np.testing.assert_array_equal(pl[SAMPLES].cpu().numpy(), epl)
    np.testing.assert_array_equal(pu[SAMPLES].cpu().numpy(), epu)
    yl2, yu2 = torch.empty_like(out), torch.empty_like(out)
    _C.conv_bound_inf_dist_forward_nograd(lo, up, wd, yl2, yu2, *geo)
    assert torch.equal(yl, yl2) and torch.equal(yu, yu2)
    assert bool((yl <= out).all()) and bool((out <= yu).all())
    del yl2, yu2
    gxl, gxu = torch.full_like(imd, float("nan")), torch.full_like(imd, float("nan"))
    gw = torch.full_like(wd, float("nan"))
    _C.conv_bound_inf_dist_backward_input_weight(gd, g2d, pl, pu, gxl, gxu, gw, *geo)
    exl_p, exu_p, _ = O.bound_inf_dist_backward(g.numpy()[SAMPLES], g2.numpy()[SAMPLES], epl, epu, 1152)
    fold = lambda a: F.fold(torch.from_numpy(a.astype(np.float64)), (32, 32), 3, 1, 1, 1).numpy()
    assert_close(gxl[SAMPLES].cpu().numpy(), fold(exl_p), what="fused conv grad_lower")
    assert_close(gxu[SAMPLES].cpu().numpy(), fold(exu_p), what="fused conv grad_upper")
    ew = (_scatter_weight_gradient(g.numpy(), pl.cpu().numpy(), 128, 1152, skip_code=0xffffffff)
          + _scatter_weight_gradient(g2.numpy(), pu.cpu().numpy(), 128, 1152))
    assert_close(gw.cpu().numpy(), ew, what="fused conv grad_weight (bounds)")


def test_conv_shape_finite_p_entry_points(monkeypatch):
    # The conv benchmark at p = 8 through the image entry points (reference: F.unfold + norm_dist::forward /
    # backward_input_weight, core/modules/norm_dist.py:93-102).  Oracle on the patches of three samples: values and
    # grad_input of those samples through the adjoint of unfold; grad_weight of those three samples alone from a
    # second call.  Over all 128 samples: the degree-1 homogeneity of the distance,
    # <grad_x, x> + <grad_w, w> = <grad_out, out> (patches are linear in the image), the sum of grad_weight over the
    # two halves of the batch, and the two routes of the backward (patches gathered inside the kernel; patches written
    # out as rows first) giving the same grad_input bit for bit when they walk the batch in the same parts.
    from core import _C
    import torch.nn.functional as F
    gen = torch.Generator().manual_seed(2022)
    img = torch.randn(128, 128, 32, 32, generator=gen)
    w = torch.randn(128, 1152, generator=gen) / np.sqrt(1152)
    g = torch.randn(128, 128, 1024, generator=gen)
    SAMPLES = [0, 63, 127]
    P = 8.0
    geo = (1, P, 3, 1, 1, 1)  # groups, p, kernel, dilation, padding, stride
    imd, wd, gd = img.cuda(), w.cuda(), g.cuda()
    patches = F.unfold(img[SAMPLES], 3, 1, 1, 1).numpy()
    out = torch.empty(128, 128, 1024, device="cuda")
    _C.conv_norm_dist_forward(imd, wd, out, *geo)
    assert_close(out[SAMPLES].cpu().numpy(), O.norm_dist_forward(patches, w.numpy(), P), what="conv p=8 forward")
    gx = torch.full_like(imd, float("nan"))
    gw = torch.full_like(wd, float("nan"))
    _C.conv_norm_dist_backward_input_weight(gd, imd, wd, out, gx, gw, *geo)
    ex_p, ew3 = O.norm_dist_backward(g.numpy()[SAMPLES], patches, w.numpy(), out[SAMPLES].cpu().numpy(), P)
    ex = F.fold(torch.from_numpy(ex_p), (32, 32), 3, 1, 1, 1).numpy()
    assert_close(gx[SAMPLES].cpu().numpy(), ex, what="conv p=8 grad_input")
    sel = torch.tensor(SAMPLES, device="cuda")
    gx3 = torch.full((3, 128, 32, 32), float("nan"), device="cuda")
    gw3 = torch.full_like(wd, float("nan"))
    _C.conv_norm_dist_backward_input_weight(gd[sel].contiguous(), imd[sel].contiguous(), wd, out[sel].contiguous(),
                                            gx3, gw3, *geo)
    assert_close(gw3.cpu().numpy(), ew3, what="conv p=8 grad_weight of three samples")
    assert_close(gx3.cpu().numpy(), ex, what="conv p=8 grad_input of three samples")
    lhs = (gx.double() * imd.double()).sum().item() + (gw.double() * wd.double()).sum().item()
    rhs = (gd.double() * out.double()).sum().item()
    scale = (gd.double().abs() * out.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-6 * scale, (lhs, rhs, scale)
    halves = torch.zeros_like(wd, dtype=torch.float64)
    for h in (slice(0, 64), slice(64, 128)):
        gxh, gwh = torch.full_like(imd[h], float("nan")), torch.full_like(wd, float("nan"))
        _C.conv_norm_dist_backward_input_weight(gd[h], imd[h], wd, out[h], gxh, gwh, *geo)
        assert torch.equal(gxh, gx[h])
        halves += gwh.double()
    assert_close(gw.cpu().numpy(), halves.cpu().numpy(), what="conv p=8 grad_weight over the halves of the batch")
    # (the order of the sums over the output channels depends on how many rows a launch covers: same parts, same bits)
    monkeypatch.setenv("NORM_DIST_CONV_PART_MB", "128")  # doubled where the kernel gathers: three parts of 43 samples
    gx_three = torch.full_like(imd, float("nan"))
    _C.conv_norm_dist_backward_input_weight(gd, imd, wd, out, gx_three, torch.empty_like(wd), *geo)
    assert_close(gx_three.cpu().numpy(), gx.cpu().numpy(), what="conv p=8 grad_input, three parts")
    monkeypatch.setenv("NORM_DIST_CONV_PART_MB", "256")  # the default: three parts for the route with two buffers
    monkeypatch.setenv("NORM_DIST_BWD_GATHER", "0")
    gx_rows, gw_rows = torch.full_like(imd, float("nan")), torch.full_like(wd, float("nan"))
    _C.conv_norm_dist_backward_input_weight(gd, imd, wd, out, gx_rows, gw_rows, *geo)
    assert torch.equal(gx_rows, gx_three)
    assert_close(gw_rows.cpu().numpy(), gw.cpu().numpy(), what="conv p=8 grad_weight, patches as rows")


def test_config4_mlp_step_full_size():
    # MLPModel(depth 6, width 5120) on [512, 3072] uniform inputs, p = 8, hinge loss on the worst-case margins of random
    # labels (reference: ell_inf_models.py:16-46, main.py:304-310): one full forward + backward step.  Every layer's
    # operator call is recorded and checked against the oracle on sampled rows (forward, grad_input) and on a slice
    # of output features (grad_weight); the degree-1 homogeneity of the distance gives an identity over ALL elements
    # of each layer (<grad_x, x> + <grad_w, w> = <grad_out, out>); mean shift, margins and loss are recomputed in
    # float64 from the recorded tensors.
    import sys
    from ell_inf_models import MLPModel, hinge
    torch.manual_seed(2021)
    model = MLPModel(depth=6, width=5120, input_dim=(3, 32, 32), identity_val=10.0).cuda()
    for m in model.modules():
        if hasattr(m, "p"):
            m.p = 8.0
    x = torch.rand(512, 3, 32, 32, device="cuda")
    t = torch.randint(0, 10, (512,), device="cuda")
    eps = 8 / 255 / 0.2009
    mod = sys.modules["core.modules.norm_dist"]
    orig = mod.norm_dist
    calls = []

    def recording(inp, w, p, groups=1, tag=None):
        inp = inp.detach().requires_grad_(True) if not inp.requires_grad else inp
        out = orig(inp, w, p, groups, tag=tag)
        rec = {"x": inp, "w": w, "out": out}
        inp.register_hook(lambda gr, rec=rec: rec.__setitem__("gx", gr.detach().clone()))
        out.register_hook(lambda gr, rec=rec: rec.__setitem__("g", gr.detach().clone()))
        calls.append(rec)
        return out

    mod.norm_dist = recording
    try:
        logits, margin = model(x, targets=t, eps=eps)
        loss = hinge()(logits, margin, t)
        loss.backward()
    finally:
        mod.norm_dist = orig
    torch.cuda.synchronize()
    assert [tuple(c["w"].shape) for c in calls] == [(5120, 3072)] + [(5120, 5120)] * 4 + [(10, 5120)]
    rows = [0, 31, 32, 255, 256, 383, 500, 511]
    cols = slice(1000, 1064)
    for li, c in enumerate(calls):
        xs, ws, outs = c["x"].detach(), c["w"].detach(), c["out"].detach()
        g, gx, gw = c["g"], c["gx"], c["w"].grad
        xn, wn, on, gn = (a.cpu().numpy() for a in (xs, ws, outs, g))
        assert_close(on[rows], O.norm_dist_forward(xn[rows], wn, 8.0), what="layer %d forward rows" % li)
        # The mean shift of the next layer makes every column of grad_output sum to zero, and the identity
        # initialisation gives every output one dominant term (|t| / out close to 1): grad_weight is then a sum of
        # terms that cancel to about 1e-5 of their size, and a float32 evaluation of the terms cannot be better than
        # that amplification allows.  Tolerance: 1e-5, or twice the error of the plain float32 yardstick where that
        # yardstick itself misses 1e-5.
        ex, _ = O.norm_dist_backward(gn[rows], xn[rows], wn, on[rows], 8.0, with_weight=False)
        tol, _ = backward_tolerances(gn[rows], xn[rows], wn, on[rows], 8.0, 1, ex, None)
        assert_close(gx.cpu().numpy()[rows], ex, tol=tol, what="layer %d grad_input rows" % li)
        cs = cols if ws.shape[0] > 64 else slice(0, ws.shape[0])
        _, ew = O.norm_dist_backward(gn[:, cs], xn, wn[cs], on[:, cs], 8.0)
        _, tol = backward_tolerances(gn[:, cs], xn, wn[cs], on[:, cs], 8.0, 1, None, ew)
        print("layer %d: grad_weight tolerance %.2e" % (li, tol))
        assert_close(gw.cpu().numpy()[cs], ew, tol=tol, what="layer %d grad_weight slice" % li)
        lhs = float((gx.double() * xs.double()).sum() + (gw.double() * ws.double()).sum())
        rhs = float((g.double() * outs.double()).sum())
        assert abs(lhs - rhs) <= 1e-5 * max(abs(rhs), float((g.double() * outs.double()).abs().sum()) * 1e-2), (li, lhs, rhs)
    # between the operator calls: batch-mean shift (hidden layers), bias (last layer); then the margin tail and the loss
    for li in range(5):
        shifted = calls[li]["out"].detach().double()
        shifted = shifted - shifted.mean(dim=(0, 2), keepdim=True)
        assert rel_err(calls[li + 1]["x"].detach().cpu().numpy(), shifted.cpu().numpy()) < 1e-5
    last = model.fc_dist[-1]
    dist = (calls[-1]["out"].detach().double().squeeze(-1) + last.bias.detach().double()).cpu().numpy()
    assert rel_err(logits.detach().cpu().numpy(), -dist) < 1e-6
    lower, upper = -(dist + eps), -(dist - eps)
    tt = t.cpu().numpy()
    m64 = upper - lower[np.arange(512), tt][:, None]
    m64[np.arange(512), tt] = 0.0
    m64 /= 2 * eps
    assert rel_err(margin.detach().cpu().numpy(), m64) < 1e-5
    res = np.maximum(m64, 0.0)
    loss64 = 0.75 * res.max(axis=1).mean() + 0.25 * res.mean()
    assert abs(loss.item() - loss64) <= 1e-5 * max(1.0, abs(loss64))


def test_config4_mlp_step_full_size_at_p_inf():
    # The same stack at p = inf, the exponent the reference's schedule ends on and the one certification uses:
    # every layer's operator call recorded, its forward compared with the oracle over EVERY output (bit-exact
    # values; the codes through the gradients they route), its backward with the oracle's scatter from the
    # oracle's own codes.  The layers are identity-initialised, so the library's default path selects the hot
    # k-tiles by the rows of w.
    import sys
    from ell_inf_models import MLPModel, hinge
    torch.manual_seed(2021)
    model = MLPModel(depth=6, width=5120, input_dim=(3, 32, 32), identity_val=10.0).cuda()
    for m in model.modules():
        if hasattr(m, "p"):
            m.p = float("inf")
    x = torch.rand(512, 3, 32, 32, device="cuda")
    t = torch.randint(0, 10, (512,), device="cuda")
    eps = 8 / 255 / 0.2009
    mod = sys.modules["core.modules.norm_dist"]
    orig = mod.norm_dist
    calls = []

    def recording(inp, w, p, groups=1, tag=None):
        inp = inp.detach().requires_grad_(True) if not inp.requires_grad else inp
        out = orig(inp, w, p, groups, tag=tag)
        rec = {"x": inp, "w": w, "out": out}
        inp.register_hook(lambda gr, rec=rec: rec.__setitem__("gx", gr.detach().clone()))
        out.register_hook(lambda gr, rec=rec: rec.__setitem__("g", gr.detach().clone()))
        calls.append(rec)
        return out

    mod.norm_dist = recording
    try:
        logits, margin = model(x, targets=t, eps=eps)
        loss = hinge()(logits, margin, t)
        loss.backward()
    finally:
        mod.norm_dist = orig
    torch.cuda.synchronize()
    assert [tuple(c["w"].shape) for c in calls] == [(5120, 3072)] + [(5120, 5120)] * 4 + [(10, 5120)]
    for li, c in enumerate(calls):
        xn, wn = c["x"].detach().cpu().numpy(), c["w"].detach().cpu().numpy()
        eo, ep = O.inf_dist_forward(xn, wn)
        np.testing.assert_array_equal(c["out"].detach().cpu().numpy(), eo, err_msg="layer %d forward" % li)
        gn = c["g"].cpu().numpy()
        ex, ew = O.inf_dist_backward(gn, ep, xn.shape[1])
        assert_close(c["gx"].cpu().numpy(), ex, what="layer %d grad_input" % li)
        # grad_weight: on these layers every batch row of an output names the same planted weight, and behind a mean
        # shift the grad_output of an output sums to zero over the batch: the exact gradient is (nearly) zero
        # everywhere, a sum of 512 terms that cancel.  The error is therefore measured against the size of what is
        # summed, not against the (vanishing) result.
        scale = float(np.abs(gn).sum(axis=(0, 2)).max())
        err = float(np.abs(c["w"].grad.cpu().numpy().astype(np.float64) - ew).max())
        assert err <= 1e-5 * scale, "layer %d grad_weight: error %.3e against terms summing to %.3e" % (li, err, scale)
    assert torch.isfinite(loss)
