"""Thin end-to-end harness around the distance-neuron operators, one batch at a time: a wrapper that routes an
input (and, for certification, its interval) through a feature net and a head, one optimisation step, a
projected-gradient attack, and the certified-accuracy evaluation.  The reference's loops over a data loader,
its logging and its schedules are not part of this package.

Same public names, signatures and results as the reference's model/model.py:3-29 (Model, set_eps, get_eps),
attack.py:4-36 (AttackPGD), main.py:60-105 (train) and main.py:166-194 (certified_test).
"""
import contextlib

import torch
import torch.nn as nn
import torch.nn.functional as F

from .norm_dist import get_p_norm, set_p_norm


def _box(x, lo, hi):
    """x clipped elementwise into [lo, hi] (tensors or numbers that broadcast)."""
    return torch.minimum(torch.maximum(x, torch.as_tensor(lo, dtype=x.dtype, device=x.device)),
                         torch.as_tensor(hi, dtype=x.dtype, device=x.device))


class Model(nn.Module):
    """`feature` maps (x, lower, upper) to such a triple; `predictor` turns the triple (and the targets) into the
    outputs.  Bounds only travel when targets are given; if the feature net produced none (or there is no feature
    net), the head gets the eps-ball around the features."""

    def __init__(self, feature, predictor, eps):
        super().__init__()
        self.feature, self.predictor, self.eps = feature, predictor, eps

    def forward(self, x, lower=None, upper=None, targets=None):
        certify = targets is not None
        triple = (x, lower if certify else None, upper if certify else None)
        if self.feature is not None:
            triple = self.feature(triple[0], lower=triple[1], upper=triple[2])
        feat, lo, hi = triple
        if certify and (lo is None or hi is None):
            lo, hi = feat - self.eps, feat + self.eps
        return self.predictor(feat, lo, hi, targets=targets)


def _wrappers(model):
    return (m for m in model.modules() if isinstance(m, Model))


def set_eps(model, eps):
    for wrapper in _wrappers(model):
        wrapper.eps = eps


def get_eps(model):
    return next((wrapper.eps for wrapper in _wrappers(model)), None)


def cal_acc(outputs, targets):
    return outputs.argmax(dim=1).eq(targets).float()


def train_step(net, loss_fun, optimizer, inputs, targets):
    """One optimisation step; returns (loss, accuracy) of the batch.  net(inputs, targets=targets) gives
    (outputs, worse_outputs); loss_fun takes them and the targets."""
    net.train()
    outputs, worse_outputs = net(inputs, targets=targets)
    loss = loss_fun(outputs, worse_outputs, targets)
    optimizer.zero_grad()
    loss.backward()
    optimizer.step()
    return loss.item(), cal_acc(outputs.detach(), targets).mean().item()


@contextlib.contextmanager
def _frozen(net):
    """Parameters take no gradient inside the block; their flags come back afterwards."""
    flags = {p: p.requires_grad for p in net.parameters()}
    net.requires_grad_(False)
    try:
        yield
    finally:
        for p, flag in flags.items():
            p.requires_grad_(flag)


class AttackPGD:
    """Signed-gradient ascent on the summed cross entropy, projected after every step onto the L_inf ball of
    radius eps around the inputs and onto the data range [down, up].  random_start: a clipped Gaussian offset
    (std eps/4, at most eps/2) first."""

    def __init__(self, net, eps, step_size, num_steps, up, down, random_start=True):
        self.net, self.eps, self.step_size, self.num_steps = net, eps, step_size, num_steps
        self.up, self.down, self.rand = up, down, random_start

    def _project(self, x, centre=None):
        if centre is not None:
            x = _box(x, centre - self.eps, centre + self.eps)
        return _box(x, self.down, self.up)

    def find(self, inputs, targets):
        start = inputs.detach()
        if self.rand:
            offset = torch.empty_like(start).normal_(0, self.eps / 4).clamp_(-self.eps / 2, self.eps / 2)
            start = self._project(start + offset)
        adv = start
        with _frozen(self.net):
            for _ in range(self.num_steps):
                adv = adv.detach().requires_grad_(True)
                F.cross_entropy(self.net(adv), targets, reduction="sum").backward()
                adv = self._project(adv.detach() + self.step_size * adv.grad.sign(), centre=inputs)
        return adv.detach()


@torch.no_grad()
def certified_accuracy(net, inputs, targets, eps, up, down):
    """Fraction of the batch whose prediction is certified for every perturbation of L_inf size eps: the interval
    bounds go through the net at p = inf, and the worst-case margins must still favour the label."""
    keep = (get_p_norm(net), get_eps(net), net.training)
    set_eps(net, eps)
    set_p_norm(net, float("inf"))
    net.eval()
    try:
        # the lower corner is clipped from below only and the upper corner from above only (reference main.py:178-179)
        lower = torch.maximum(inputs - eps, torch.as_tensor(down, dtype=inputs.dtype, device=inputs.device))
        upper = torch.minimum(inputs + eps, torch.as_tensor(up, dtype=inputs.dtype, device=inputs.device))
        worst = net(inputs, lower=lower, upper=upper, targets=targets)[1]
        return cal_acc(worst, targets).mean().item()
    finally:
        set_p_norm(net, keep[0])
        set_eps(net, keep[1])
        net.train(keep[2])
