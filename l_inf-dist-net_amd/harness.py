"""Thin end-to-end harness around the distance-neuron operators: the model wrapper, a training step, the PGD
attack and the certified-accuracy evaluation of the reference, for one batch at a time (the reference's loops
over a data loader, its logging and its schedules are not part of this package).

Reference: model/model.py:3-29 (Model, set_eps, get_eps), attack.py:4-36 (AttackPGD), main.py:60-105 (train),
main.py:166-194 (certified_test).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .norm_dist import get_p_norm, set_p_norm


class Model(nn.Module):
    """feature (a dist net returning (y, lower, upper)) followed by predictor (a head taking them plus targets)."""

    def __init__(self, feature, predictor, eps):
        super().__init__()
        self.feature = feature
        self.predictor = predictor
        self.eps = eps

    def forward(self, x, lower=None, upper=None, targets=None):
        if targets is None:
            lower = upper = None
        if self.feature is not None:
            x, lower, upper = self.feature(x, lower=lower, upper=upper)
        if targets is not None and (lower is None or upper is None):
            lower = x - self.eps
            upper = x + self.eps
        return self.predictor(x, lower, upper, targets=targets)


def set_eps(model, eps):
    for m in model.modules():
        if isinstance(m, Model):
            m.eps = eps


def get_eps(model):
    for m in model.modules():
        if isinstance(m, Model):
            return m.eps
    return None


def cal_acc(outputs, targets):
    return (outputs.max(dim=1)[1] == targets).float()


def train_step(net, loss_fun, optimizer, inputs, targets):
    """One optimisation step as the reference's training loop makes it; returns (loss, accuracy) of the batch.
    net(inputs, targets=targets) gives (outputs, worse_outputs); loss_fun takes them and the targets."""
    net.train()
    outputs, worse_outputs = net(inputs, targets=targets)
    loss = loss_fun(outputs, worse_outputs, targets)
    optimizer.zero_grad()
    loss.backward()
    optimizer.step()
    with torch.no_grad():
        return loss.item(), cal_acc(outputs, targets).mean().item()


class AttackPGD:
    """Projected gradient ascent on the cross entropy inside the eps-ball (L_inf) around the inputs, clipped to
    the data range [down, up]."""

    def __init__(self, net, eps, step_size, num_steps, up, down, random_start=True):
        self.net, self.eps, self.step_size, self.num_steps = net, eps, step_size, num_steps
        self.up, self.down, self.rand = up, down, random_start

    def find(self, inputs, targets):
        saved = [p.requires_grad for p in self.net.parameters()]
        self.net.requires_grad_(False)
        x = inputs.detach()
        if self.rand:
            noise = torch.zeros_like(x).normal_(0, self.eps / 4)
            x = x + torch.clamp(noise, -self.eps / 2, self.eps / 2)
            x = torch.min(torch.max(x, self.down), self.up)
        for _ in range(self.num_steps):
            x.requires_grad_()
            loss = F.cross_entropy(self.net(x), targets, reduction="sum")
            loss.backward()
            x = torch.add(x.detach(), torch.sign(x.grad.detach()), alpha=self.step_size)
            x = torch.min(torch.max(x, inputs - self.eps), inputs + self.eps)
            x = torch.min(torch.max(x, self.down), self.up)
        for p, r in zip(self.net.parameters(), saved):
            p.requires_grad_(r)
        return x


@torch.no_grad()
def certified_accuracy(net, inputs, targets, eps, up, down):
    """Fraction of the batch whose prediction is certified for every perturbation of L_inf size eps: the interval
    bounds go through the net at p = inf, and the worst-case margins must still favour the label."""
    save_p, save_eps = get_p_norm(net), get_eps(net)
    set_eps(net, eps)
    set_p_norm(net, float("inf"))
    was_training = net.training
    net.eval()
    lower = torch.max(inputs - eps, down)
    upper = torch.min(inputs + eps, up)
    worst = net(inputs, lower=lower, upper=upper, targets=targets)[1]
    res = cal_acc(worst, targets).mean().item()
    set_p_norm(net, save_p)
    set_eps(net, save_eps)
    net.train(was_training)
    return res
