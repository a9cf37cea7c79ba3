"""The convolutional L_inf-dist net of the reference (model/conv.py:6-31): five 3x3 NormDistConv layers with mean
shift (width, width, then 2*width with a stride-2 layer in front), one hidden NormDist layer and a NormDist head.
On the GPU at p = inf every conv layer here runs from the image (no unfolded tensor): the 3-channel first layer
with its channels resident in LDS, the wide ones staged four channels at a time.
"""
import torch.nn as nn

from .norm_dist import NormDist, NormDistConv

net_width = 32


def _negated(triple):
    """(-y, -upper, -lower): the net's outputs are negated distances, which exchanges the two bounds."""
    y, lo, up = triple
    return [None if t is None else -t for t in (y, up, lo)]


class Conv(nn.Module):
    # (out channels as a multiple of the base width, stride) of the five 3x3 layers
    PLAN = ((1, 1), (1, 1), (2, 2), (2, 1), (2, 1))

    def __init__(self, width, input_dim, hidden=512, num_classes=10):
        super().__init__()
        base = width * net_width
        channels, height, wide = input_dim
        layers, c_in = [], channels
        for mult, stride in self.PLAN:
            layers.append(NormDistConv(c_in, mult * base, 3, stride=stride, padding=1, bias=False, mean_normalize=True))
            c_in = mult * base
            height, wide = (height + stride - 1) // stride, (wide + stride - 1) // stride
        self.conv = nn.ModuleList(layers)
        self.fc = NormDist(height * wide * c_in, hidden, bias=False, mean_normalize=True)
        self.fc_last = NormDist(hidden, num_classes, bias=True, mean_normalize=False)

    def forward(self, x, lower=None, upper=None):
        triple = (x, lower, upper)
        for layer in self.conv:
            triple = layer(*triple)
        flat = [None if t is None else t.flatten(1) for t in triple]
        return _negated(self.fc_last(*self.fc(*flat)))
