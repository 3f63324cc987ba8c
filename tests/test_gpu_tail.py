"""The fused tail of the distance network: worst-case margins and the hinge loss on them against the reference's
formulation in torch primitives, evaluated in float64 (ell_inf_models.py:41-46, main.py:304-310): values and
gradients, with and without interval bounds, and through the model."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _reference(x, lower, upper, targets, eps, mix):
    if lower is None:
        lower, upper = x - eps, x + eps
    x, lower, upper = -x, -upper, -lower
    idx = targets.view(-1, 1)
    margin = (upper - torch.gather(lower, 1, idx)).scatter(1, idx, 0) / (2 * eps)
    res = margin.clamp(min=0)
    return margin, (1 - mix) * res.max(dim=1)[0].mean() + mix * res.mean()


@pytest.mark.parametrize("bounds", [False, True])
@pytest.mark.parametrize("B,C", [(512, 10), (37, 7), (1500, 100)])
def test_margins_and_hinge(B, C, bounds):
    from core.norm_dist import hinge_loss, worst_margin
    gen = torch.Generator().manual_seed(B + C)
    x = torch.randn(B, C, generator=gen) * 0.3 + 2.0
    radius = torch.rand(B, C, generator=gen) * 0.05
    targets = torch.randint(0, C, (B,), generator=gen)
    eps, mix = 8 / 255, 0.25
    leaves64 = [t.double().requires_grad_(True) for t in ((x - radius, x + radius) if bounds else (x,))]
    if bounds:
        m64, l64 = _reference(torch.zeros_like(leaves64[0]), leaves64[0], leaves64[1], targets, eps, mix)
    else:
        m64, l64 = _reference(leaves64[0], None, None, targets, eps, mix)
    l64.backward()
    leaves = [t.detach().float().cuda().requires_grad_(True) for t in leaves64]
    tg = targets.cuda()
    if bounds:
        margin = worst_margin(None, leaves[0], leaves[1], tg, eps)
    else:
        margin = worst_margin(leaves[0], None, None, tg, eps)
    loss = hinge_loss(margin, mix)
    loss.backward()
    # (1e-5 of the largest margin: the division by 2 eps amplifies the float32 rounding of x[t] - x[c] sixteen times)
    assert (margin.detach().cpu().double() - m64.detach()).abs().max().item() <= 1e-5 * m64.abs().max().item()
    assert abs(loss.item() - l64.item()) <= 1e-5 * abs(l64.item()) + 1e-7
    for got, want in zip(leaves, leaves64):
        scale = want.grad.abs().max().item()
        assert (got.grad.cpu().double() - want.grad).abs().max().item() <= 1e-5 * scale + 1e-12
    # repeated calls give the same bits (sums in a fixed order)
    assert torch.equal(hinge_loss(margin.detach(), mix), hinge_loss(margin.detach(), mix))


def test_model_tail_matches_torch_primitives():
    """MLPModel's (logits, margins) and the hinge on them equal the torch-primitive formulation on the same network
    output."""
    from ell_inf_models import MLPModel, hinge
    torch.manual_seed(1)
    model = MLPModel(depth=3, width=64, input_dim=(1, 8, 8), identity_val=10.0).cuda()
    img = torch.rand(48, 1, 8, 8, device="cuda")
    lab = torch.randint(0, 10, (48,), device="cuda")
    eps = 0.1
    out, worst = model(img, targets=lab, eps=eps)
    loss = hinge()(out, worst, lab)
    dist = -out.detach() / (model.scalar if isinstance(model.scalar, int) else model.scalar.detach())
    m, l = _reference(dist.double(), None, None, lab, eps, 0.25)
    assert (worst.detach().double() - m).abs().max().item() <= 1e-5 * m.abs().max().item()
    assert abs(loss.item() - l.item()) <= 1e-5 * abs(l.item()) + 1e-7
    loss.backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


def test_label_outside_the_classes_gives_nan_rows_not_a_fault():
    from core import _C
    x = torch.randn(6, 10, device="cuda")
    t = torch.tensor([0, 9, 10, -1, 3, 4], device="cuda")
    m = torch.empty_like(x)
    _C.margin_forward(x, None, None, t, 0.1, m)
    bad = torch.isnan(m).all(dim=1).cpu()
    assert bad.tolist() == [False, False, True, True, False, False]
    gx = torch.full_like(x, 7.0)
    _C.margin_backward(torch.ones_like(x), t, 0.1, gx, None, None)
    assert torch.isfinite(gx).all()


def test_nan_margins_reach_the_loss_as_in_the_torch_formula():
    """clamp(min=0).max().mean() of the reference's loss (main.py:304-310) propagates NaN: a NaN margin (diverged
    activations, the NaN row of an out-of-range label) must give a NaN loss, not a finite one; the gradient of the
    NaN entries is what torch's clamp / max backward give them."""
    from core.norm_dist import hinge_loss
    torch.manual_seed(7)
    margin = torch.randn(12, 10, device="cuda")
    margin[3, 4] = float("nan")
    margin[8] = float("nan")
    for mix in (0.25, 0.0, 1.0):
        a = margin.clone().requires_grad_(True)
        b = margin.clone().requires_grad_(True)
        loss = hinge_loss(a, mix)
        res = b.clamp(min=0)
        want = (1 - mix) * res.max(dim=1)[0].mean() + mix * res.mean()
        assert torch.isnan(loss) and torch.isnan(want)
        loss.backward()
        want.backward()
        assert torch.equal(torch.isnan(a.grad), torch.isnan(b.grad))
        # finite everywhere else, and zero on the NaN entries themselves (masked by relu's derivative)
        assert torch.isfinite(a.grad).all() and float(a.grad[8].abs().sum()) == 0.0 and float(a.grad[3, 4]) == 0.0
    clean = torch.randn(12, 10, device="cuda")
    assert torch.isfinite(hinge_loss(clean, 0.25))
