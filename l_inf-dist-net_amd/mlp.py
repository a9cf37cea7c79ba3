"""The fully connected L_inf-dist net that the operator benchmarks are quoted on.

Reference: model/mlp.py:7-23 (MLP) and model/bound_module.py:95-103
(BoundFinalIdentity).  Hidden layers are NormDist with mean shift and no bias;
the head is a NormDist with bias.  The output triple is negated, which swaps the
roles of the lower and upper bound.
"""
import numpy as np
import torch
import torch.nn as nn

from .norm_dist import NormDist

net_width = 1024


class MLP(nn.Module):
    def __init__(self, depth, width, input_dim, num_classes=10, head_mean_normalize=False):
        super().__init__()
        dim = int(np.prod(input_dim))
        layers = []
        for _ in range(depth - 1):
            layers.append(NormDist(dim, net_width * width, bias=False, mean_normalize=True))
            dim = net_width * width
        self.fc = nn.ModuleList(layers)
        self.fc_last = NormDist(dim, num_classes, bias=True, mean_normalize=head_mean_normalize)

    def forward(self, x, lower=None, upper=None):
        triple = [None if t is None else t.flatten(1) for t in (x, lower, upper)]
        for layer in (*self.fc, self.fc_last):
            triple = layer(*triple)
        y, lo, up = triple
        return [None if t is None else -t for t in (y, up, lo)]   # negated distances: the bounds change places


class BoundFinalIdentity(nn.Module):
    """Certified margins: res[b, j] = upper[b, j] - lower[b, target_b], res[b, target_b] = 0."""

    def forward(self, x, lower=None, upper=None, targets=None):
        if lower is None or upper is None or targets is None:
            return x
        at = targets.view(-1, 1)
        margins = upper - lower.gather(1, at)          # every class's upper bound against the label's lower bound
        return x, margins.scatter(1, at, 0.0)
