"""A short training run in which the schedule moves the exponent at every iteration, from p = 8 through general p to
p = infinity, on one model: the operator dispatches on p at run time, so nothing is compiled or cached per exponent;
every step must leave finite losses and gradients, and the exponent set on the layers must be the one the operator
uses (reference: main.py:262-299, 357)."""
import math

import pytest
import torch

from core.norm_dist import norm_dist
from ell_inf_models import MLPModel, hinge
from schedule import TrainingSchedule, get_normdist_models

pytestmark = pytest.mark.gpu


def test_exponent_changes_every_iteration():
    torch.manual_seed(3)
    model = MLPModel(depth=4, width=256, input_dim=(1, 16, 16), num_classes=10).cuda()
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    sch = TrainingSchedule((0, 0, 0, 3, 4), 6, model, opt, p_start=8.0, p_end=1000.0, eps_train=0.1)  # full radius from the start
    loss_fn = hinge()
    x = torch.rand(64, 1, 16, 16, device="cuda")
    t = torch.randint(0, 10, (64,), device="cuda")
    seen = []
    for epoch in range(4):
        for it in range(6):
            eps, p, lam, lr = sch(epoch, it)
            seen.append(p)
            out, worst = model(x, targets=t, eps=eps)
            loss = loss_fn(out, worst, t)
            opt.zero_grad()
            loss.backward()
            assert math.isfinite(loss.item())
            assert all(torch.isfinite(q.grad).all() for q in model.parameters() if q.grad is not None)
            opt.step()
    assert seen[0] == 8.0 and math.isinf(seen[-1]) and len(set(seen)) >= 19
    layer = get_normdist_models(model)[0]
    for p in (8.0, 11.3, 77.0, float("inf")):
        layer.p = p
        y = torch.rand(5, 256, device="cuda")
        direct = norm_dist(y.unsqueeze(-1), layer.weight, p, layer.groups).squeeze(-1)
        layer.eval()
        got = layer(y)[0]
        shift = layer.mean_shift.running_mean if layer.mean_shift is not None else 0
        assert torch.allclose(got + shift, direct, rtol=1e-6, atol=1e-6)
