"""The trainer-side schedule (exponent, radius, learning rate), the loss heads beside the hinge and checkpoint loading,
pinned by what the definitions fix: end points and the geometric midpoint of the exponent ramp, the switch to
p = infinity, the cosine and step learning rates, value and slope continuity of the smooth radius ramp at its joint,
and round trips of state dicts with and without the data-parallel prefix (reference: main.py:244-300, 313-334,
394-410)."""
import math
from types import SimpleNamespace

import pytest
import torch

from core.modules import NormDist
from ell_inf_models import MLPModel
from schedule import TrainingSchedule, adapt_state_dict, create_schedule, crossentropy, get_normdist_models, \
    load_checkpoint, mixture


def _setup(**kw):
    model = MLPModel(depth=3, width=16, input_dim=(1, 4, 4), num_classes=10)
    opt = torch.optim.Adam([{"params": model.parameters(), "lr": 0.02}, {"params": [torch.zeros(1, requires_grad=True)], "lr": 0.5}])
    args = dict(epochs=(2, 6, 1, 9, 12), batch_per_epoch=50, model=model, optimizer=opt, p_start=8.0, p_end=1000.0,
                eps_train=0.3)
    args.update(kw)
    return model, opt, TrainingSchedule(**args)


def test_exponent_ramp_and_layers():
    model, opt, sch = _setup()
    layers = get_normdist_models(model)
    assert len(layers) == 3 and all(isinstance(m, NormDist) for m in layers)
    assert sch.p_norm(0) == 8.0 and sch.p_norm(1) == 8.0           # before the ramp
    assert math.isclose(sch.p_norm(5), math.sqrt(8.0 * 1000.0), rel_tol=1e-12)  # half way: geometric mean
    assert math.isclose(sch.p_norm(8, 49), 8.0 * 125.0 ** (399 / 400), rel_tol=1e-12)  # counted in iterations
    assert sch.p_norm(9) == float("inf") and sch.p_norm(11, 3) == float("inf")
    eps, p, lam, lr = sch(5, 0)
    assert all(m.p == p for m in layers) and lam == 0
    _, _, sch2 = _setup(p_end=64.0)  # an end point below 100 is kept, not replaced by infinity
    assert math.isclose(sch2.p_norm(11), 64.0, rel_tol=1e-12)


def test_learning_rates():
    model, opt, sch = _setup()
    sch(0, 0)
    assert [g["lr"] for g in opt.param_groups] == [0.02, 0.5]
    sch(6, 0)
    assert math.isclose(opt.param_groups[0]["lr"], 0.01, rel_tol=1e-12)  # half of the cosine
    assert math.isclose(opt.param_groups[1]["lr"], 0.25, rel_tol=1e-12)
    sch(12, 0)
    assert abs(opt.param_groups[0]["lr"]) < 1e-17
    model, opt, sch = _setup(decays="4,8")
    assert [round(sch(e, 0)[3] / 0.02, 12) for e in (0, 3, 4, 7, 8, 11)] == [1, 1, 0.2, 0.2, 0.04, 0.04]


def test_radius_ramps():
    _, _, lin = _setup()
    assert lin.eps(2) == 0 and math.isclose(lin.eps(4), 0.15) and lin.eps(6) == 0.3 and lin.eps(10) == 0.3
    _, _, sm = _setup(eps_schedule="smooth", eps_smooth=0.4)
    assert sm.eps(2) == 0 and math.isclose(sm.eps(6), 0.3, rel_tol=1e-12)
    # value and slope continuous where the quartic meets the line (ratio 0.4 = epoch 3.6 -> iteration 80 of 200)
    def at(it):
        return sm.eps(2 + it // 50, it % 50) / 0.3
    assert abs(at(80) - (at(79) + at(81)) / 2) < 1e-4
    left, right = at(80) - at(79), at(81) - at(80)
    assert abs(left - right) < 0.02 * right
    r = 0.4
    k = 1 / ((4 - 3 * r) * r ** 3)
    assert math.isclose(at(40), k * 0.2 ** 4, rel_tol=1e-12)
    with pytest.raises(NotImplementedError):
        _setup(eps_schedule="cubic")


def test_mixture_weight_follows_the_exponent_ramp():
    loss = mixture(lam0=0.1, lam_end=0.001)
    _, _, sch = _setup(loss=loss)
    assert sch(1, 0)[2] == 0.1
    assert math.isclose(sch(5, 0)[2], 0.01, rel_tol=1e-12)
    assert math.isclose(sch(9, 0)[2], 0.001, rel_tol=1e-12)
    out = torch.tensor([[2.0, 0.0, -1.0], [0.0, 1.0, 0.5]])
    worst = torch.tensor([[0.0, 3.0, -2.0], [0.2, 0.0, 0.7]])
    t = torch.tensor([0, 1])
    ce = torch.nn.functional.cross_entropy(out, t)
    assert torch.allclose(loss(out, worst, t), torch.tensor((1.0 + 0.7) / 2) + 0.001 * ce)
    cw = torch.nn.functional.cross_entropy(worst, t)
    assert torch.allclose(crossentropy(0.25)(out, worst, t), 0.75 * cw + 0.25 * ce)


def test_create_schedule_reads_the_reference_argument_names():
    model, opt, _ = _setup()
    args = SimpleNamespace(epochs=[0, 1, 0, 2, 3], decays=None, p_start=8.0, p_end=1000.0, eps_train=0.1, eps_smooth=0.0)
    sch = create_schedule(args, 10, model, opt, None)
    eps, p, lam, lr = sch(1, 0)
    assert eps == 0.1 and math.isclose(p, math.sqrt(8000.0), rel_tol=1e-12)


def test_checkpoint_round_trip_with_and_without_prefix(tmp_path):
    model, opt, _ = _setup()
    sd = model.state_dict()
    wrapped = adapt_state_dict(sd, parallel=True)
    assert all(k.startswith("module.") for k in wrapped)
    assert list(adapt_state_dict(wrapped, parallel=False)) == list(sd)
    assert adapt_state_dict(sd, parallel=False) is sd
    path = tmp_path / "ckpt.pth"
    torch.save({"state_dict": dict(wrapped), "optimizer": opt.state_dict()}, path)
    other, opt2, _ = _setup()
    with torch.no_grad():
        for q in other.parameters():
            q.add_(1.0)
    load_checkpoint(str(path), other, opt2)
    for a, b in zip(model.state_dict().values(), other.state_dict().values()):
        assert torch.equal(a, b)
