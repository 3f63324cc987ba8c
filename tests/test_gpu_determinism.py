"""Run-to-run reproducibility of the finite-p backward (reference: norm_dist::backward_input is deterministic for
grad_input, core/cuda/norm_dist_cuda.cu:246-334).  grad_input of the row-split kernel is a fixed-order sum: blocks
that two workgroups share go through a buffer and are added in workgroup order.  grad_weight is a fixed-order sum
while the batch is one row chunk.  Checked bit for bit on repeated calls, on shapes that split blocks between
workgroups (many co units per slab), that do not (few), with several row chunks, groups and the conv layout."""
import numpy as np
import pytest
import torch

from util import dev

pytestmark = pytest.mark.gpu

SHAPES = [  # B, CO, CI, G, HW, grad_weight reproducible too
    (512, 2048, 640, 1, 1, True),     # 128 co units per slab: every block is shared by several workgroups
    (512, 48, 5120, 1, 1, True),      # 3 co units per slab: most blocks have one owner, some are split
    (300, 200, 333, 1, 1, False),     # three 128-row chunks, ragged slab
    (50, 320, 700, 1, 1, True),       # 64-row configuration
    (256, 200, 333, 1, 1, True),      # one 256-row workgroup per block, ragged slab
    (1000, 160, 320, 1, 1, False),    # two row chunks: grad_weight adds with atomics
    (600, 128, 1024, 2, 1, False),    # groups, five 128-row chunks
    (2, 40, 1200, 2, 64, True),       # conv layout: through the transposed copies
]


@pytest.mark.parametrize("p", [2.0, 8.0, 3.5])
@pytest.mark.parametrize("B,CO,CI,G,HW,w_too", SHAPES)
def test_backward_is_reproducible(B, CO, CI, G, HW, w_too, p):
    from core import _C
    r = np.random.RandomState(B + CO)
    x = dev(r.randn(B, CI, HW).astype(np.float32))
    w = dev((r.randn(CO, CI // G) / np.sqrt(CI // G)).astype(np.float32))
    g = dev(r.randn(B, CO, HW).astype(np.float32))
    out = torch.empty(B, CO, HW, device="cuda")
    _C.norm_dist_forward(x, w, out, G, p)
    results = []
    for _ in range(3):
        gx = torch.full_like(x, float("nan"))
        gw = torch.full_like(w, float("nan"))
        _C.norm_dist_backward_input_weight(g, x, w, out, gx, gw, G, p)
        results.append((gx, gw))
    gx2 = torch.full_like(x, float("nan"))
    _C.norm_dist_backward_input(g, x, w, out, gx2, G, p)
    assert not torch.isnan(results[0][0]).any() and not torch.isnan(results[0][1]).any()
    for gx, gw in results[1:]:
        assert torch.equal(gx, results[0][0]), "grad_input differs between two runs"
        if w_too:
            assert torch.equal(gw, results[0][1]), "grad_weight differs between two runs"
    assert torch.equal(gx2, results[0][0]), "grad_input of the input-only entry point differs"
