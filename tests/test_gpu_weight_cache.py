"""The p = inf forwards with the pre-pass over the weights kept between calls (ndist_weight_cache_prepare and the
*_nograd_cached entry points): bit-identical to the plain entry points, on problems that use the pre-pass (hot
k-tiles, k-tile skipping) and on problems that ignore it; and the layers' opt-in use of it (freeze_weights): nothing
is kept unless asked, and what is kept is checked against the oracle through every kind of weight update."""
import numpy as np
import pytest
import torch

from core import _C
from core.modules import NormDist, freeze_weights, unfreeze_weights
from oracle import norm_dist_oracle as O

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


def _oracle_triple(layer, x, lo, up):
    w = layer.weight.detach().cpu().numpy()
    a = lambda t: t.detach().cpu().numpy()[:, :, None]
    y = O.inf_dist_forward(a(x), w, with_pos=False)[0]
    yl, yu, _, _ = O.bound_inf_dist_forward(a(lo), a(up), w, with_pos=False)
    return [torch.from_numpy(t[:, :, 0]) for t in (y, yl, yu)]


def _certify(layer, x, lo, up):
    with torch.no_grad():
        return [t.cpu() for t in layer(x, lo, up)]


def _same(got, want):
    return all(torch.equal(a, b) for a, b in zip(got, want))


def test_layers_keep_nothing_unless_asked():
    """Evaluation without gradients keeps no state between calls by default (like the reference's layers): weights
    rewritten through `.data`, which advances no version counter, are seen by the next certified evaluation."""
    torch.manual_seed(1)
    layer = NormDist(1024, 1024, bias=False, mean_shift=False, identity_val=10.0).cuda().eval()
    x = torch.randn(256, 1024, device="cuda")
    lo, up = x - 0.1, x + 0.1
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up))
    assert layer._weight_cache._buffer is None
    version = layer.weight._version
    layer.weight.data.mul_(-0.5)                      # e.g. weight averaging, clipping, a hand-written update
    layer.weight.data[:, :7] += 3.0
    assert layer.weight._version == version           # invisible to torch
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up))
    with torch.no_grad():
        assert torch.equal(layer(x)[0].cpu(), _oracle_triple(layer, x, lo, up)[0])


def test_frozen_weights_contract():
    """freeze_weights(): the pre-pass is kept and reused; visible updates redo it; after a `.data` write the caller
    freezes again; train(), load_state_dict() and device moves unfreeze."""
    torch.manual_seed(2)
    layer = NormDist(1024, 1024, bias=False, mean_shift=False, identity_val=10.0).cuda().eval()
    x = torch.randn(256, 1024, device="cuda")
    lo, up = x - 0.1, x + 0.1
    cache = layer._weight_cache
    assert layer.freeze_weights() and cache.frozen
    buffer = cache._buffer
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up)) and cache._buffer is buffer
    with torch.no_grad():
        assert torch.equal(layer(x)[0].cpu(), _oracle_triple(layer, x, lo, up)[0]) and cache._buffer is buffer
        layer.weight.add_(torch.randn_like(layer.weight))          # an optimizer-style update: version advances
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up)) and cache._buffer is not buffer
    layer.weight.data.mul_(-0.5)                                   # invisible: the contract asks for a new freeze
    layer.freeze_weights()
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up))
    layer.train()
    assert not cache.frozen and cache._buffer is None
    layer.eval()
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up)) and cache._buffer is None
    layer.freeze_weights()
    layer.load_state_dict({"weight": torch.randn(1024, 1024)})
    assert not cache.frozen
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up))
    layer.freeze_weights()
    layer.float()                                                  # any _apply (moves, casts) unfreezes
    assert not cache.frozen
    layer.freeze_weights()
    with torch.enable_grad():                                      # with gradients the kept pre-pass is not used
        layer(x)[0].sum().backward()
    assert "_weight_cache" not in layer.state_dict()
    model = torch.nn.Sequential(layer, NormDist(1024, 64).cuda())
    model.eval()
    assert freeze_weights(model) == 2 and model[1]._weight_cache.frozen
    unfreeze_weights(model)
    assert not layer._weight_cache.frozen and not model[1]._weight_cache.frozen


def test_non_contiguous_weights_are_never_cached():
    torch.manual_seed(3)
    layer = NormDist(640, 1280, bias=False, mean_shift=False).cuda().eval()
    with torch.no_grad():
        layer.weight = torch.nn.Parameter(torch.randn(640, 1280, device="cuda").t())   # [1280, 640], strided
    assert not layer.weight.is_contiguous()
    assert layer.freeze_weights() is False and not layer._weight_cache.frozen
    x = torch.randn(200, 640, device="cuda")
    lo, up = x - 0.1, x + 0.1
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up))
    layer.weight.data.mul_(2.0)
    assert _same(_certify(layer, x, lo, up), _oracle_triple(layer, x, lo, up))


def test_cache_size_and_validation():
    import ctypes
    lib = ctypes.CDLL(_C.LIBRARY_PATH)
    lib.ndist_weight_cache_bytes.restype = ctypes.c_longlong
    assert lib.ndist_weight_cache_bytes(5120, 5120, 1) == 4 * 5120 * (2 + 160)
    assert lib.ndist_weight_cache_bytes(0, 5120, 1) == 0
    assert lib.ndist_weight_cache_bytes(8, 10, 4) == 0      # CI not divisible by G
