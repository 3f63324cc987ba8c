"""The p = inf forwards with the pre-pass over the weights kept between calls (ndist_weight_cache_prepare and the
*_nograd_cached entry points): bit-identical to the plain entry points, on problems that use the pre-pass (hot
k-tiles, k-tile skipping) and on problems that ignore it; and the layer's use of it in evaluation: the cache follows
the weights through in-place updates and moves."""
import numpy as np
import pytest
import torch

from core import _C
from core.modules import NormDist

pytestmark = pytest.mark.gpu


def _data(B, CO, CI, G, kind, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, CI, 1, generator=g)
    w = torch.randn(CO, CI // G, generator=g)
    if kind == "small_w":      # a few k-tiles per row of x decide every maximum
        w /= CI ** 0.5
    elif kind == "diagonal":   # one planted entry per row of w
        w *= 0.3
        w[torch.arange(CO), torch.arange(CO) % (CI // G)] = -10.0
    return x.cuda(), w.cuda()


@pytest.mark.parametrize("kind", ["small_w", "diagonal", "dense"])
@pytest.mark.parametrize("B,CO,CI,G", [(256, 1024, 1024, 1), (64, 2048, 4096, 2), (300, 640, 1280, 1), (7, 40, 96, 1)])
def test_cached_forwards_are_bit_identical(B, CO, CI, G, kind):
    x, w = _data(B, CO, CI, G, kind, B + CO)
    xl, xu = x - 0.05, x + 0.05
    cache = _C.weight_cache(w, G)
    ref = torch.empty(B, CO, 1, device="cuda")
    got = torch.empty_like(ref)
    _C.inf_dist_forward_nograd(x, w, ref, G)
    _C.inf_dist_forward_nograd_cached(x, w, cache, got, G)
    assert torch.equal(ref, got)
    r = [torch.empty_like(ref) for _ in range(3)]
    c = [torch.empty_like(ref) for _ in range(3)]
    _C.inf_and_bound_forward_nograd(x, xl, xu, w, r[0], r[1], r[2], G)
    _C.inf_and_bound_forward_nograd_cached(x, xl, xu, w, cache, c[0], c[1], c[2], G)
    for a, b in zip(r, c):
        assert torch.equal(a, b)
    assert torch.equal(r[0], ref)


def test_layer_cache_follows_the_weights():
    torch.manual_seed(1)
    layer = NormDist(1024, 1024, bias=False, mean_shift=False).cuda().eval()
    x = torch.randn(256, 1024, device="cuda")

    def plain():
        out = torch.empty(256, 1024, 1, device="cuda")
        _C.inf_dist_forward_nograd(x.unsqueeze(-1).contiguous(), layer.weight.detach(), out, 1)
        return out.squeeze(-1)

    with torch.no_grad():
        first = layer(x)[0]
        assert torch.equal(first, plain())
        buffer = layer._weight_cache._buffer
        assert buffer is not None
        assert torch.equal(layer(x)[0], first) and layer._weight_cache._buffer is buffer  # kept
        layer.weight.add_(torch.randn_like(layer.weight))                                 # an optimizer-style update
        assert torch.equal(layer(x)[0], plain()) and layer._weight_cache._buffer is not buffer
        buffer = layer._weight_cache._buffer
        layer.load_state_dict({"weight": torch.randn(1024, 1024)})
        assert torch.equal(layer(x)[0], plain()) and layer._weight_cache._buffer is not buffer
        lo, up = x - 0.1, x + 0.1
        y, yl, yu = layer(x, lo, up)
        r = [torch.empty(256, 1024, 1, device="cuda") for _ in range(3)]
        _C.inf_and_bound_forward_nograd(*(t.unsqueeze(-1).contiguous() for t in (x, lo, up)), layer.weight.detach(), *r, 1)
        assert all(torch.equal(a, b.squeeze(-1)) for a, b in zip((y, yl, yu), r))
    layer.train()
    before = layer._weight_cache._key
    layer(x)          # training: the cache is left alone
    assert layer._weight_cache._key == before
    assert "_weight_cache" not in layer.state_dict()


def test_cache_size_and_validation():
    import ctypes
    lib = ctypes.CDLL(_C.LIBRARY_PATH)
    lib.ndist_weight_cache_bytes.restype = ctypes.c_longlong
    assert lib.ndist_weight_cache_bytes(5120, 5120, 1) == 4 * 5120 * (2 + 160)
    assert lib.ndist_weight_cache_bytes(0, 5120, 1) == 0
    assert lib.ndist_weight_cache_bytes(8, 10, 4) == 0      # CI not divisible by G
