"""Calls share no state but idle scratch arenas, handed to one call at a time: host threads on their own streams may
call the library concurrently
(reference: stateless kernels, core/cuda/norm_dist.cpp; the binding here adds the caller's stream)."""
import threading

import pytest
import torch

pytestmark = pytest.mark.gpu


def _one(seed, p, repeat, results, errors):
    try:
        from core.norm_dist import norm_dist
        gen = torch.Generator().manual_seed(seed)
        x = torch.randn(64, 300, 1, generator=gen).cuda()
        w = (torch.randn(90, 300, generator=gen) / 17).cuda()
        g = torch.randn(64, 90, 1, generator=gen).cuda()
        stream = torch.cuda.Stream()
        outs = []
        with torch.cuda.stream(stream):
            for _ in range(repeat):
                xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
                y = norm_dist(xr, wr, p)
                y.backward(g)
                outs.append((y.detach(), xr.grad, wr.grad))
        stream.synchronize()
        results[seed] = outs
    except Exception as e:  # surfaced by the main thread
        errors.append(e)


@pytest.mark.parametrize("p", [8.0, float("inf"), 13.7])
def test_concurrent_callers_on_their_own_streams(p):
    serial, errors = {}, []
    for seed in range(4):
        _one(seed, p, 1, serial, errors)
    assert not errors, errors
    results = {}
    threads = [threading.Thread(target=_one, args=(seed, p, 10, results, errors)) for seed in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
    for seed in range(4):
        y0, gx0, gw0 = serial[seed][0]
        for y, gx, gw in results[seed]:
            assert torch.equal(y, y0)  # the forward is deterministic
            # float atomics: the order of summation may differ from run to run, also without threads
            assert float((gx - gx0).abs().max()) <= 1e-5 * float(gx0.abs().max())
            assert float((gw - gw0).abs().max()) <= 1e-5 * float(gw0.abs().max())


def test_mode_overrides_belong_to_the_calling_thread():
    """ndist_set_skip_mode / hot_mode / scaled_mode change the calling thread's settings only: a thread that forces
    kernel variants (a test, a tuning run) cannot leave other callers on another kernel path."""
    from core import _C
    base = _C.get_modes()
    seen = {}

    def other():
        seen["before"] = _C.get_modes()
        _C.set_skip_mode(1, 0)
        _C.set_hot_mode(3)
        _C.set_scaled_mode(0)
        seen["after"] = _C.get_modes()

    t = threading.Thread(target=other)
    t.start()
    t.join(30)
    assert seen["before"] == base and seen["after"] == (1, 0, 3, 0)
    assert _C.get_modes() == base                      # untouched here
    _C.set_hot_mode(2)
    try:
        assert _C.get_modes()[2] == 2
        t = threading.Thread(target=lambda: seen.__setitem__("fresh", _C.get_modes()))
        t.start()
        t.join(30)
        assert seen["fresh"] == base                   # a new thread starts from the environment's values
    finally:
        _C.set_hot_mode(-1)
    assert _C.get_modes() == base
