"""The entry point that allocates nothing (ndist_norm_dist_backward_input_weight_noalloc, no counterpart in the
reference): called through the C ABI, checked against the allocating entry point it is a variant of (bit for bit
where that path sums in a fixed order, to 1e-5 where it uses atomics) and against the float64 oracle, on two calls in a
row, the second with a smaller input; the library's own allocation counters must not move across the calls; and
recorded into a HIP graph, which is what such callers do with it."""
import numpy as np
import pytest
import torch

import oracle.norm_dist_oracle as O
from util import assert_close

pytestmark = pytest.mark.gpu

REL = 1e-5  # the tolerance of every finite-p gradient of the operator


def _inputs(seed, B, CO, CI, HW=1, G=1):
    r = np.random.RandomState(seed)
    x = r.randn(B, CI, HW).astype(np.float32)
    w = (r.randn(CO, CI // G) / np.sqrt(CI // G)).astype(np.float32)
    g = r.randn(B, CO, HW).astype(np.float32)
    return x, w, g


def _both(x, w, g, p, G=1):
    """grad_input, grad_weight of the allocating entry point and of the no-allocation one, for the same forward."""
    from core import _C
    xt, wt, gt = (torch.from_numpy(a).cuda() for a in (x, w, g))
    out = torch.empty(x.shape[0], w.shape[0], x.shape[2], device="cuda")
    _C.norm_dist_forward(xt, wt, out, G, p)
    gx0, gw0 = torch.empty_like(xt), torch.empty_like(wt)
    _C.norm_dist_backward_input_weight(gt, xt, wt, out, gx0, gw0, G, p)
    # poison the outputs of the call under test: it must overwrite every element
    gx1, gw1 = torch.full_like(xt, float("nan")), torch.full_like(wt, float("nan"))
    torch.cuda.synchronize()
    before = _C.scratch_counters()
    _C.norm_dist_backward_input_weight_noalloc(gt, xt, wt, out, gx1, gw1, G, p)
    torch.cuda.synchronize()
    assert _C.scratch_counters() == before, "the no-allocation entry point went to the allocator"
    return out, (gx0, gw0), (gx1, gw1)


def _compare(x, w, g, p, G, out, ref, got, what):
    assert_close(got[0].cpu().numpy(), ref[0].cpu().numpy(), tol=REL, what=what + " grad_input vs allocating entry point")
    assert_close(got[1].cpu().numpy(), ref[1].cpu().numpy(), tol=REL, what=what + " grad_weight vs allocating entry point")
    # up to 128 rows are one row chunk: grad_weight is summed in a fixed order by both, identical bits
    if x.shape[0] * x.shape[2] <= 128:
        assert torch.equal(got[1], ref[1]), what + ": grad_weight differs bitwise"
    ex, ew = O.norm_dist_backward(g, x, w, out.cpu().numpy(), p, G)
    assert_close(got[0].cpu().numpy(), ex, tol=REL, what=what + " grad_input vs oracle")
    assert_close(got[1].cpu().numpy(), ew, tol=REL, what=what + " grad_weight vs oracle")


@pytest.mark.parametrize("p", [8.0, 3.0, 13.7, 1.5])
def test_two_calls_in_a_row_the_second_smaller(p):
    big = _inputs(5, 300, 200, 520)
    small = _inputs(6, 70, 48, 130)
    # the first call leaves its factors all over the shared array; the second must not see them
    for name, (x, w, g) in (("first (300x200x520)", big), ("second, smaller (70x48x130)", small)):
        out, ref, got = _both(x, w, g, p)
        _compare(x, w, g, p, 1, out, ref, got, "p=%g %s" % (p, name))


def test_groups_conv_layout_and_repeat():
    x, w, g = _inputs(7, 6, 24, 36, HW=50, G=3)
    out, ref, got = _both(x, w, g, 8.0, G=3)
    _compare(x, w, g, 8.0, 3, out, ref, got, "groups, HW=50")
    out2, ref2, got2 = _both(x, w, g, 8.0, G=3)
    assert_close(got2[0].cpu().numpy(), got[0].cpu().numpy(), tol=REL, what="repeat grad_input")
    assert_close(got2[1].cpu().numpy(), got[1].cpu().numpy(), tol=REL, what="repeat grad_weight")


def test_headline_shape_fits_and_larger_is_refused():
    from core import _C
    assert _C.noalloc_scratch_bytes() >= 512 * 5120 * 4
    # 4096 x 5120 needs 80 MiB of factors: refused with its own status before anything is launched
    B, CO, CI = 4096, 5120, 64
    x = torch.zeros(B, CI, 1, device="cuda")
    w = torch.zeros(CO, CI, device="cuda")
    out = torch.ones(B, CO, 1, device="cuda")
    g = torch.zeros_like(out)
    gx = torch.full_like(x, 7.0)
    gw = torch.full_like(w, 7.0)
    with pytest.raises(_C.NormDistError) as e:
        _C.norm_dist_backward_input_weight_noalloc(g, x, w, out, gx, gw, 1, 8.0)
    assert e.value.status == _C.ERR_TOO_LARGE
    torch.cuda.synchronize()
    assert float(gx.min()) == 7.0 and float(gw.min()) == 7.0  # untouched


def test_captured_into_a_graph_and_replayed():
    """One call of the no-allocation entry point recorded into a HIP graph (its whole purpose), replayed several
    times with eager work and synchronisations in between; every replay is compared with the allocating entry
    point on the inputs the replay saw.  A capture that starts before the array's address is known is refused."""
    from core import _C
    assert _C._lib.ndist_noalloc_prepare() == 0
    x, w, g = _inputs(11, 300, 200, 520)
    xt, wt, gt = (torch.from_numpy(a).cuda() for a in (x, w, g))
    out = torch.empty(300, 200, 1, device="cuda")
    gx, gw = torch.full_like(xt, float("nan")), torch.full_like(wt, float("nan"))
    _C.norm_dist_forward(xt, wt, out, 1, 8.0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print("capturing", flush=True)
    with torch.cuda.graph(graph):
        _C.norm_dist_backward_input_weight_noalloc(gt, xt, wt, out, gx, gw, 1, 8.0)
    torch.cuda.synchronize()
    for it in range(3):
        print("replay", it, flush=True)
        if it:  # new inputs in the captured buffers, written by eager work between the replays
            xt.copy_(torch.from_numpy(_inputs(20 + it, 300, 200, 520)[0]).cuda())
            gt.mul_(-0.5)
            _C.norm_dist_forward(xt, wt, out, 1, 8.0)
        gx.fill_(float("nan"))
        gw.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rx, rw = torch.empty_like(xt), torch.empty_like(wt)
        _C.norm_dist_backward_input_weight(gt, xt, wt, out, rx, rw, 1, 8.0)
        torch.cuda.synchronize()
        assert_close(gx.cpu().numpy(), rx.cpu().numpy(), tol=REL, what="replay %d grad_input" % it)
        assert_close(gw.cpu().numpy(), rw.cpu().numpy(), tol=REL, what="replay %d grad_weight" % it)
    del graph
