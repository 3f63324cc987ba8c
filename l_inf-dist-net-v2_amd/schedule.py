"""Host-side glue a trainer needs around the distance layers: the per-iteration schedule of the exponent p, the
perturbation radius and the learning rate, the two remaining loss heads, and checkpoint loading that accepts state
dicts saved with or without the `module.` prefix of a data-parallel wrapper.

Reference: main.py:240-300 (create_schedule), main.py:313-334 (crossentropy, mixture), main.py:394-410 (checkpoint).
The exponent changes at every iteration; the library dispatches on p at run time (no per-exponent compilation, no
cache to warm), so setting `layer.p` is all a step has to do.
"""
import bisect
import math
from collections import OrderedDict

import torch
import torch.nn.functional as F

from core.modules import NormDistBase


def get_normdist_models(model):
    """The distance layers of a model (main.py:240-241)."""
    return [m for m in model.modules() if isinstance(m, NormDistBase)]


class TrainingSchedule:
    """schedule(epoch, minibatch) -> (eps, p, lam, lr); sets the learning rates of `optimizer`, the exponent of every
    distance layer of `model` and, when the loss has an `update(ratio)` method, its mixing weight.

    epochs = (eps_start, eps_end, p_start, p_end, total): epochs at which the radius and the exponent begin and
    finish their ramps.  Progress inside a ramp is counted in iterations:
        ratio = clip((epoch - start) * batches + minibatch) / ((end - start) * batches), 0, 1), 1 for an empty ramp.
    p   = p_start * (p_end / p_start)^ratio, and infinity once the ramp is complete if p_end >= 100;
    lr  = lr0 / 5^(number of decay epochs passed) with `decays`, else half a cosine over the whole run;
    eps = eps_train * ratio ('linear'), or the 'smooth' ramp: quartic k * ratio^4 up to ratio = r, then the straight
          line through (1, 1) that continues it with the same value and slope, k = 1 / ((4 - 3 r) r^3).
    """

    def __init__(self, epochs, batch_per_epoch, model, optimizer, loss=None, p_start=8.0, p_end=1000.0, eps_train=0.0,
                 decays=None, eps_schedule="linear", eps_smooth=0.0):
        self.eps_epochs, self.p_epochs, self.total = (epochs[0], epochs[1]), (epochs[2], epochs[3]), epochs[4]
        self.batches = batch_per_epoch
        self.layers = get_normdist_models(model)
        self.optimizer = optimizer
        self.loss = loss
        self.p_start, self.p_end, self.eps_train = float(p_start), float(p_end), float(eps_train)
        if isinstance(decays, str):
            decays = [int(e) for e in decays.split(",")]
        self.decays = decays
        if eps_schedule not in ("linear", "smooth"):
            raise NotImplementedError(eps_schedule)
        self.eps_schedule, self.eps_smooth = eps_schedule, float(eps_smooth)
        self.base_lrs = [group["lr"] for group in optimizer.param_groups]

    def ratio(self, epoch, start, end, minibatch=0):
        if end <= start:
            return 1
        done = (epoch - start) * self.batches + minibatch
        return min(max(done / ((end - start) * self.batches), 0), 1)

    def p_norm(self, epoch, minibatch=0):
        r = self.ratio(epoch, *self.p_epochs, minibatch)
        if r >= 1 and self.p_end >= 100:
            return float("inf")
        return self.p_start * math.exp(math.log(self.p_end / self.p_start) * r)

    def eps(self, epoch, minibatch=0):
        r = self.ratio(epoch, *self.eps_epochs, minibatch)
        s = self.eps_smooth
        if self.eps_schedule == "linear" or s == 0:
            return self.eps_train * r
        k = 1 / ((4 - 3 * s) * s ** 3)
        if r < s:
            return k * r ** 4 * self.eps_train
        return ((1 - k * s ** 4) / (1 - s) * (r - 1) + 1) * self.eps_train

    def lr_factor(self, epoch, minibatch=0):
        if self.decays is None:
            return 0.5 * (1 + math.cos(self.ratio(epoch, 0, self.total, minibatch) * math.pi))
        return 1 / 5 ** bisect.bisect_right(self.decays, epoch)

    def __call__(self, epoch, minibatch):
        f = self.lr_factor(epoch, minibatch)
        for group, lr in zip(self.optimizer.param_groups, self.base_lrs):
            group["lr"] = f * lr
        p = self.p_norm(epoch, minibatch)
        for layer in self.layers:
            layer.p = p
        lam = 0
        if hasattr(self.loss, "update"):
            self.loss.update(self.ratio(epoch, *self.p_epochs, minibatch))
            lam = self.loss.lam
        return self.eps(epoch, minibatch), p, lam, self.optimizer.param_groups[0]["lr"]


def create_schedule(args, batch_per_epoch, model, optimizer, loss, eps_schedule="linear"):
    """The reference's entry point (main.py:244): `args` carries epochs, decays, p_start, p_end, eps_train and
    eps_smooth as its argument parser names them."""
    return TrainingSchedule(args.epochs, batch_per_epoch, model, optimizer, loss, args.p_start, args.p_end,
                            args.eps_train, args.decays, eps_schedule, args.eps_smooth)


class crossentropy:
    """(1 - mix) * CE(worst-case logits) + mix * CE(clean logits) (main.py:313-318)."""

    def __init__(self, mix=0):
        self.mix = mix

    def __call__(self, outputs, worst_outputs, targets):
        return (1 - self.mix) * F.cross_entropy(worst_outputs, targets) + self.mix * F.cross_entropy(outputs, targets)


class mixture:
    """Clipped hinge on the worst-case margins plus lam * CE(clean logits), lam decaying geometrically from lam0 to
    lam_end along the exponent's ramp (main.py:321-334)."""

    def __init__(self, lam0=0.1, lam_end=0.001, clip=1):
        self.lam_start, self.lam_end, self.lam, self.clip = lam0, lam_end, lam0, clip

    def update(self, ratio):
        self.lam = self.lam_start * (self.lam_end / self.lam_start) ** ratio

    def __call__(self, outputs, worst_outputs, targets):
        worst = worst_outputs.clamp(min=0, max=self.clip).max(dim=1)[0].mean()
        return worst + self.lam * F.cross_entropy(outputs, targets)


def adapt_state_dict(state_dict, parallel):
    """Adds or strips the `module.` prefix so that a state dict saved from a wrapped model loads into a bare one and
    the reverse (main.py:401-406)."""
    wrapped = next(iter(state_dict)).startswith("module.")
    if wrapped and not parallel:
        return OrderedDict((k[len("module."):], v) for k, v in state_dict.items())
    if not wrapped and parallel:
        return OrderedDict(("module." + k, v) for k, v in state_dict.items())
    return state_dict


def load_checkpoint(path, model, optimizer=None, parallel=False, map_location="cpu"):
    """Loads a checkpoint of the reference's layout ({'state_dict': ..., 'optimizer': ...}, main.py:394-410) with a
    loader that executes nothing from the file."""
    checkpoint = torch.load(path, map_location=map_location, weights_only=True)
    model.load_state_dict(adapt_state_dict(checkpoint["state_dict"], parallel))
    if optimizer is not None and "optimizer" in checkpoint:
        optimizer.load_state_dict(checkpoint["optimizer"])
    return checkpoint
