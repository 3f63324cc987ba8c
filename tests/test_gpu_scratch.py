"""Temporary device memory of the library: arenas kept per (device, stream) and reused call after call instead of
stream-ordered allocations (no counterpart in the reference, whose temporaries come from PyTorch's caching allocator).
Results must not depend on what an arena held before: growing shapes, shrinking shapes, two streams, release."""
import numpy as np
import pytest
import torch

import oracle.norm_dist_oracle as O
from util import assert_close

pytestmark = pytest.mark.gpu


def _case(seed, B, CO, CI, p):
    r = np.random.RandomState(seed)
    x = r.randn(B, CI, 1).astype(np.float32)
    w = (r.randn(CO, CI) / np.sqrt(CI)).astype(np.float32)
    g = r.randn(B, CO, 1).astype(np.float32)
    out = O.norm_dist_forward(x, w, p).astype(np.float32)
    ex, ew = O.norm_dist_backward(g, x, w, out, p)
    return x, w, g, out, ex, ew


def _run(case, p, stream=None):
    from core import _C
    x, w, g, out, ex, ew = case
    with torch.cuda.stream(stream or torch.cuda.current_stream()):
        xt, wt, gt = (torch.from_numpy(a).cuda() for a in (x, w, g))
        ot = torch.empty(x.shape[0], w.shape[0], 1, device="cuda")
        gx, gw = torch.empty_like(xt), torch.empty_like(wt)
        _C.norm_dist_forward(xt, wt, ot, 1, p)
        _C.norm_dist_backward_input_weight(gt, xt, wt, ot, gx, gw, 1, p)
    return ot, gx, gw


def _check(res, case, what):
    ot, gx, gw = res
    torch.cuda.synchronize()
    assert_close(ot.cpu().numpy(), case[3], what=what + " forward")
    assert_close(gx.cpu().numpy(), case[4], what=what + " grad_input")
    assert_close(gw.cpu().numpy(), case[5], what=what + " grad_weight")


@pytest.mark.parametrize("p", [8.0, 13.7, 40.0])
def test_growing_and_shrinking_requests_reuse_the_arena(p):
    from core import _C
    _C.set_skip_mode(1, 1)  # p = 40: the variants with probe and seed scratch, also on these small problems
    try:
        shapes = [(70, 40, 300), (300, 130, 700), (33, 20, 2048), (600, 64, 512), (70, 40, 300)]
        cases = [_case(11 + i, B, CO, CI, p) for i, (B, CO, CI) in enumerate(shapes)]
        results = [_run(c, p) for c in cases]  # queued back to back: later calls reuse the bytes of earlier ones
        for i, (res, c) in enumerate(zip(results, cases)):
            _check(res, c, "call %d %s" % (i, shapes[i]))
        _C.release_scratch()
        _check(_run(cases[1], p), cases[1], "after release")
    finally:
        _C.set_skip_mode(-1, -1)


def test_two_streams_have_their_own_arenas():
    p = 13.7
    a, b = _case(3, 200, 96, 640, p), _case(4, 130, 50, 1000, p)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    res = []
    for _ in range(4):  # interleaved on the host, concurrent on the device
        res.append((_run(a, p, s1), a))
        res.append((_run(b, p, s2), b))
    for i, (r, c) in enumerate(res):
        _check(r, c, "interleaved call %d" % i)


def test_warmed_up_calls_allocate_nothing():
    """Once an arena has grown to what its stream needs, calls with scratch neither allocate nor free (which is
    also why they do not wait for the device): the library's own count of hipMalloc / hipFree calls stands still."""
    from core import _C
    B, CO, CI, p = 256, 1024, 1024, 8.0
    x = torch.randn(B, CI, 1, device="cuda")
    w = torch.randn(CO, CI, device="cuda") / 32
    out = torch.empty(B, CO, 1, device="cuda")
    g = torch.randn_like(out)
    gx, gw = torch.empty_like(x), torch.empty_like(w)
    xs, outs, gs, gxs = x[:64].contiguous(), out[:64].contiguous(), g[:64].contiguous(), gx[:64].contiguous()
    _C.norm_dist_forward(x, w, out, 1, p)
    for _ in range(3):
        _C.norm_dist_backward_input_weight(g, x, w, out, gx, gw, 1, p)  # arena at its final size
    torch.cuda.synchronize()
    before = _C.scratch_counters()
    for _ in range(5):
        _C.norm_dist_backward_input_weight(g, x, w, out, gx, gw, 1, p)
        _C.inf_dist_forward_nograd(xs, w, outs, 1)                       # k range split over workgroups: scratch too
        _C.norm_dist_backward_input_weight(gs, xs, w, outs, gxs, gw, 1, p)  # smaller request, same arena
    torch.cuda.synchronize()
    assert _C.scratch_counters() == before
    _C.release_scratch()
    after = _C.scratch_counters()
    assert after[1] > before[1] and after[0] == before[0]  # release frees, allocates nothing


def _hip():
    import ctypes
    lib = ctypes.CDLL("libamdhip64.so")
    lib.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    lib.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
    lib.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
    lib.hipGraphDestroy.argtypes = [ctypes.c_void_p]
    lib.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    return lib, ctypes


def test_scratch_taking_calls_refuse_a_stream_under_capture():
    """A graph must not capture calls that take arena scratch (a later call may free the block whose address the
    graph holds): they return NDIST_ERR_CAPTURE before allocating or launching anything.  The capture is ended and
    the (empty) graph destroyed; nothing is instantiated or replayed."""
    from core import _C
    hip, ctypes = _hip()
    case = _case(21, 96, 40, 200, 8.0)
    x, w, g, out = (torch.from_numpy(a).cuda() for a in case[:4])
    gx = torch.full_like(x, 5.0)
    gw = torch.full_like(w, 5.0)
    torch.cuda.synchronize()
    st = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(st)) == 0
    graph = ctypes.c_void_p()
    before = _C.scratch_counters()
    assert hip.hipStreamBeginCapture(st, 1) == 0  # hipStreamCaptureModeThreadLocal
    try:
        with pytest.raises(_C.NormDistError) as e:
            _C._run(_C._norm_bwd_xw, x.device, g.data_ptr(), x.data_ptr(), w.data_ptr(), out.data_ptr(), 96, 40, 200, 1, 1,
                    gx.data_ptr(), gw.data_ptr(), 8.0, stream=st.value)
        assert e.value.status == _C.ERR_CAPTURE
    finally:
        assert hip.hipStreamEndCapture(st, ctypes.byref(graph)) == 0
        if graph.value:
            hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(st)
    torch.cuda.synchronize()
    assert _C.scratch_counters() == before
    assert float(gx.min()) == 5.0 and float(gw.min()) == 5.0  # nothing ran
    # the same call outside a capture still works
    _C.norm_dist_backward_input_weight(g, x, w, out, gx, gw, 1, 8.0)
    torch.cuda.synchronize()
    assert_close(gx.cpu().numpy(), case[4], what="after the refused call: grad_input")
    assert_close(gw.cpu().numpy(), case[5], what="after the refused call: grad_weight")
