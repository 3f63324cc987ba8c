"""Model stacks built from the distance layers (reference: ell_inf_models.py).  `MLPModel` is the shape of the
end-to-end training-step benchmark; `HybridModel` is kept for API parity."""
import math

import torch
import torch.nn as nn

from core.modules import NormDist, NormDistBase
from core.modules import BoundTanh, BoundLinear, BoundFinalLinear, BoundSequential
from core.modules import apply_if_not_none
from core.norm_dist import hinge_loss, worst_margin


def check_inf_and_eval(model):
    """True when every distance layer runs at p = inf in eval mode: the only state in which interval bounds
    can be propagated (reference: ell_inf_models.py:9-13)."""
    return all(math.isinf(m.p) and not m.training for m in model.modules() if isinstance(m, NormDistBase))


def _box(x, eps, up, down, model):
    if up is not None and down is not None and check_inf_and_eval(model):
        return x, torch.maximum(x - eps, down), torch.minimum(x + eps, up)
    return x, None, None


class hinge:
    """Hinge loss on the worst-case margins: (1 - mix) * mean_b max_c relu(m) + mix * mean relu(m)
    (reference: main.py:304-310)."""

    def __init__(self, mix=0.25):
        self.mix = mix

    def __call__(self, outputs, worst_outputs, targets):
        return hinge_loss(worst_outputs, self.mix)


class HybridModel(nn.Module):
    """Distance layers followed by a small interval-aware MLP head (reference: ell_inf_models.py:49-76)."""

    def __init__(self, depth, width, input_dim, hidden=512, num_classes=10, std=1.0, identity_val=None):
        super().__init__()
        kw = {'std': std, 'identity_val': identity_val}
        pixels = input_dim[0] * input_dim[1] * input_dim[2]
        sizes = [pixels] + [width] * (depth - 2)
        self.fc_dist = BoundSequential(*[NormDist(a, b, bias=False, mean_shift=True, **kw)
                                         for a, b in zip(sizes[:-1], sizes[1:])])
        self.fc_linear = BoundSequential(BoundLinear(width, hidden, bias=True), BoundTanh())
        self.fc_final = BoundFinalLinear(hidden, num_classes, bias=True)

    def forward(self, x=None, targets=None, eps=0, up=None, down=None):
        paras = apply_if_not_none(_box(x, eps, up, down, self), lambda t: t.view(t.size(0), -1))
        paras = self.fc_dist(paras)
        if targets is not None and (paras[1] is None or paras[2] is None):
            paras = paras[0], paras[0] - eps, paras[0] + eps
        return self.fc_final(*self.fc_linear(paras), targets=targets)


class MLPModel(nn.Module):
    """depth distance layers: pixels -> width -> ... -> width -> num_classes (reference: ell_inf_models.py:16-46).
    Returns -distance as logits; with `targets`, also the worst-case margins of a radius-`eps` ball."""

    def __init__(self, depth, width, input_dim, num_classes=10, std=1.0, identity_val=None, scalar=False):
        super().__init__()
        kw = {'std': std, 'identity_val': identity_val}
        pixels = input_dim[0] * input_dim[1] * input_dim[2]
        sizes = [pixels] + [width] * (depth - 1)
        layers = [NormDist(a, b, bias=False, mean_shift=True, **kw) for a, b in zip(sizes[:-1], sizes[1:])]
        layers.append(NormDist(width, num_classes, bias=True, mean_shift=False, **kw))
        self.fc_dist = BoundSequential(*layers)
        self.scalar = nn.Parameter(torch.ones(1)) if scalar else 1

    def forward(self, x=None, targets=None, eps=0, up=None, down=None):
        paras = apply_if_not_none(_box(x, eps, up, down, self), lambda t: t.view(t.size(0), -1))
        x, lower, upper = self.fc_dist(paras)
        if targets is None:
            return -x * self.scalar
        # logits are -x: their upper bound is -lower, the target's lower bound -upper[t]; without interval bounds the
        # network is 1-Lipschitz w.r.t. the infinity norm: lower / upper = x -/+ eps
        if (lower is None) != (upper is None):
            lower = x - eps if lower is None else lower
            upper = x + eps if upper is None else upper
        return -x * self.scalar, worst_margin(x, lower, upper, targets, eps)
