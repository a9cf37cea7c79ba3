"""The convolutional L_inf-dist net of the reference (model/conv.py:6-31): five 3x3 NormDistConv layers with mean
shift (width, width, then 2*width with a stride-2 layer in front), one hidden NormDist layer and a NormDist head.
On the GPU at p = inf every conv layer here runs from the image (no unfolded tensor): the 3-channel first layer
with its channels resident in LDS, the wide ones staged four channels at a time.
"""
import torch.nn as nn

from .norm_dist import NormDist, NormDistConv

net_width = 32


class Conv(nn.Module):
    def __init__(self, width, input_dim, hidden=512, num_classes=10):
        super().__init__()
        pixels = input_dim[1] * input_dim[2]
        width *= net_width
        layers = [NormDistConv(input_dim[0], width, 3, bias=False, mean_normalize=True, padding=1),
                  NormDistConv(width, width, 3, bias=False, mean_normalize=True, padding=1)]
        pixels //= 4
        width *= 2
        layers += [NormDistConv(width // 2, width, 3, bias=False, padding=1, stride=2, mean_normalize=True),
                   NormDistConv(width, width, 3, bias=False, padding=1, mean_normalize=True),
                   NormDistConv(width, width, 3, bias=False, padding=1, mean_normalize=True)]
        self.conv = nn.ModuleList(layers)
        self.fc = NormDist(pixels * width, hidden, bias=False, mean_normalize=True)
        self.fc_last = NormDist(hidden, num_classes, bias=True, mean_normalize=False)

    def forward(self, x, lower=None, upper=None):
        paras = (x, lower, upper)
        for layer in self.conv:
            paras = layer(*paras)
        paras = [None if y is None else y.view(y.size(0), -1) for y in paras]
        paras = self.fc(*paras)
        y, lo, up = self.fc_last(*paras)
        return [None if t is None else -t for t in (y, up, lo)]
