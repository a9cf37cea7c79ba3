"""Distance-neuron operators and layers with the reference's Python interface.

Mirrors model/norm_dist.py of the reference: ``DistF`` (autograd function),
``norm_dist`` / ``inf_dist_bound`` (functional API, including the dense
pure-torch formulas selected by ``use_custom_cuda_func=False``), ``MeanNorm``,
``NormDistConv``, ``NormDist``, ``set_p_norm`` / ``get_p_norm``.  The native
calls go through ``norm_dist_cpp`` (this package's ctypes binding of
libldist_hip.so) instead of the reference's CUDA extension.

Additions that the reference does not have: the aliases ``MeanNormDist`` and
the keyword spellings ``groups`` / ``mean_shift`` accepted by the layers.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import norm_dist_cpp


class DistF(torch.autograd.Function):
    """out = ||x - w||_p per (row, output); p = inf keeps the argmax for the backward.

    Reference: model/norm_dist.py:7-47.  x is (B, CI, HW), weight (CO, CI/group).
    """

    @staticmethod
    def forward(ctx, x, weight, group, p, tag):
        assert weight.size(1) * group == x.size(1)
        shape = (x.size(0), weight.size(0), x.size(2))
        output = torch.empty(shape, device=x.device, dtype=x.dtype)
        if math.isinf(p):
            pos = torch.empty(shape, device=x.device, dtype=torch.int32)
            norm_dist_cpp.inf_dist_forward(x, weight, output, pos, group)
            ctx.save_for_backward(x, weight, output, pos)
        elif p > 1:
            norm_dist_cpp.norm_dist_forward(x, weight, output, group, p)
            ctx.save_for_backward(x, weight, output)
        else:
            raise NotImplementedError
        ctx.group = group
        ctx.p = p
        ctx.tag = tag
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_input = grad_weight = None
        grad_output = grad_output.contiguous()
        if math.isinf(ctx.p):
            x, weight, output, pos = ctx.saved_tensors
            # the scatter kernels write every element, so no zero fill is needed here
            if ctx.needs_input_grad[0]:
                grad_input = torch.empty_like(x)
                norm_dist_cpp.inf_dist_backward_input_overwrite(grad_output, pos, grad_input, ctx.group)
            if ctx.needs_input_grad[1]:
                grad_weight = torch.empty_like(weight)
                norm_dist_cpp.inf_dist_backward_weight_overwrite(grad_output, pos, grad_weight, ctx.group)
        else:
            x, weight, output = ctx.saved_tensors
            if ctx.needs_input_grad[0]:
                grad_input = torch.empty_like(x)
                norm_dist_cpp.norm_dist_backward_input(grad_output, x, weight, output, grad_input, ctx.group, ctx.p)
            if ctx.needs_input_grad[1]:
                grad_weight = torch.zeros_like(weight)  # the kernel adds onto it
                norm_dist_cpp.norm_dist_backward_weight(grad_output, x, weight, output, grad_weight, ctx.group, ctx.p)
        return grad_input, grad_weight, None, None, None


def norm_dist(input, weight, group, p, use_custom_cuda_func=True, tag=None):
    """model/norm_dist.py:49-58.  The dense torch formula runs only when asked for explicitly."""
    if use_custom_cuda_func:
        return DistF.apply(input, weight, group, p, tag)
    y = input.view(input.size(0), group, 1, -1, input.size(2)) - weight.view(group, -1, weight.size(-1), 1)
    with torch.no_grad():
        normalize = torch.norm(y, dim=3, p=float("inf"), keepdim=True)
    y = torch.norm(y / normalize, dim=3, p=p, keepdim=True) * normalize
    return y.view(y.size(0), -1, y.size(-1))


def inf_dist_bound(input_lower, input_upper, weight, group, use_custom_cuda_func=True, tag=None):
    """model/norm_dist.py:60-76.  Returns (output_lower, output_upper); not differentiable."""
    shape = input_lower.size(0), weight.size(0), input_lower.size(2)
    if use_custom_cuda_func:
        output_lower = input_lower.new_empty(shape)
        output_upper = input_upper.new_empty(shape)
        norm_dist_cpp.inf_dist_bound_forward(input_lower, input_upper, weight, output_lower, output_upper, group)
        return output_lower, output_upper
    w = weight.view(group, -1, weight.size(-1), 1)
    y1 = input_lower.view(input_lower.size(0), group, 1, -1, input_lower.size(2)) - w
    y2 = input_upper.view(input_upper.size(0), group, 1, -1, input_upper.size(2)) - w
    abs_y1, abs_y2 = torch.abs(y1), torch.abs(y2)
    output_upper = torch.maximum(abs_y1, abs_y2).max(dim=3)[0].view(shape)
    output_lower = torch.minimum(abs_y1, abs_y2)
    output_lower[(y1 < 0) & (y2 > 0)] = 0
    output_lower = output_lower.max(dim=3)[0].view(shape)
    return output_lower, output_upper


class MeanNorm(nn.Module):
    """Subtracts the per-channel mean (batch mean when training, running mean otherwise).

    Reference: model/norm_dist.py:78-100.
    """

    def __init__(self, out_channels, momentum=0.1):
        super().__init__()
        self.out_channels = out_channels
        self.momentum = momentum
        self.register_buffer("running_mean", torch.zeros(out_channels))

    def forward(self, x):
        y = x.view(x.size(0), x.size(1), -1)
        if self.training:
            mean = y.mean(dim=-1).mean(dim=0) if x.dim() > 2 else x.mean(dim=0)
            with torch.no_grad():
                self.running_mean.mul_(1 - self.momentum).add_(mean, alpha=self.momentum)
        else:
            mean = self.running_mean
        return (y - mean.unsqueeze(-1)).view_as(x)

    def extra_repr(self):
        return f"{self.out_channels}"


class NormDistConv(nn.Module):
    """Convolution-shaped layer of distance neurons (model/norm_dist.py:102-169).

    forward(x, lower=None, upper=None) returns (y, lower', upper'); the bounds
    need p = inf and eval mode.
    """

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, group=1, p=0,
                 bias=True, mean_normalize=False, identity_init=True, groups=None, mean_shift=None):
        super().__init__()
        if groups is not None:
            group = groups
        if mean_shift is not None:
            mean_normalize = mean_shift
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.group = group
        self.p = p
        assert in_channels % group == 0
        assert out_channels % group == 0

        weight_tensor = torch.randn(out_channels, in_channels // group, kernel_size, kernel_size)
        if identity_init and in_channels <= out_channels:
            centre = kernel_size // 2
            for i in range(out_channels):
                weight_tensor[i, i % (in_channels // group), centre, centre] = -10.0
        self.weight = nn.Parameter(weight_tensor)
        self.normalize = MeanNorm(out_channels) if mean_normalize else None
        self.bias = nn.Parameter(torch.zeros(out_channels)) if bias else None

        if not hasattr(NormDistConv, "tag"):
            NormDistConv.tag = 0
        NormDistConv.tag += 1
        self.tag = NormDistConv.tag

    def _post(self, t):
        if self.normalize is not None:
            t = self.normalize(t)
        if self.bias is not None:
            t = t + self.bias.view(1, -1, 1, 1)
        return t

    def forward(self, x, lower=None, upper=None):
        h, w = x.size(2), x.size(3)
        out_h = (h + 2 * self.padding - self.kernel_size) // self.stride + 1
        out_w = (w + 2 * self.padding - self.kernel_size) // self.stride + 1
        if self.kernel_size == 1 and self.stride == 1 and self.padding == 0:
            # a 1x1 window is the identity: skip F.unfold, which launches one kernel per image
            unfold = lambda t: t.reshape(t.size(0), t.size(1), -1)
        else:
            unfold = lambda t: F.unfold(t, self.kernel_size, self.dilation, self.padding, self.stride)
        cols = unfold(x)
        weight = self.weight.view(self.weight.size(0), -1)
        y = norm_dist(cols.view(cols.size(0), cols.size(1), -1), weight, self.group, p=self.p, tag=self.tag)
        y = y.view(cols.size(0), -1, out_h, out_w)
        # MeanNorm updates its running mean on y only; the bounds below run in eval mode
        y = self._post(y)
        if lower is None or upper is None:
            return y, None, None
        assert math.isinf(self.p) and not self.training
        lower, upper = unfold(lower), unfold(upper)
        lower, upper = inf_dist_bound(lower.view(cols.size(0), cols.size(1), -1),
                                      upper.view(cols.size(0), cols.size(1), -1), weight, self.group, tag=self.tag)
        return y, self._post(lower.view_as(y)), self._post(upper.view_as(y))

    def extra_repr(self):
        s = f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, stride={self.stride}"
        if self.padding != 0:
            s += f", padding={self.padding}"
        if self.dilation != 1:
            s += f", dilation={self.dilation}"
        if self.group != 1:
            s += f", group={self.group}"
        if self.bias is None:
            s += ", bias=False"
        return s


class NormDist(NormDistConv):
    """Fully connected layer of distance neurons: a 1x1 NormDistConv on (B, C, 1, 1).

    Reference: model/norm_dist.py:171-187.
    """

    def __init__(self, in_features, out_features, p=0, bias=True, mean_normalize=False, identity_init=True,
                 mean_shift=None):
        super().__init__(in_features, out_features, 1, p=p, bias=bias, mean_normalize=mean_normalize,
                         identity_init=identity_init, mean_shift=mean_shift)

    def forward(self, x, lower=None, upper=None):
        x = x.unsqueeze(-1).unsqueeze(-1)
        lower = lower.view_as(x) if lower is not None else None
        upper = upper.view_as(x) if upper is not None else None
        x, lower, upper = super().forward(x, lower, upper)
        x = x.squeeze(-1).squeeze(-1)
        lower = lower.view_as(x) if lower is not None else None
        upper = upper.view_as(x) if upper is not None else None
        return x, lower, upper

    def extra_repr(self):
        return f"in_features={self.in_channels}, out_features={self.out_channels}, bias={self.bias is not None}"


class MeanNormDist(NormDist):
    """NormDist with the mean shift switched on (no class of this name exists in the reference)."""

    def __init__(self, in_features, out_features, p=0, bias=False, identity_init=True):
        super().__init__(in_features, out_features, p=p, bias=bias, mean_normalize=True, identity_init=identity_init)


def set_p_norm(model, p):
    """model/norm_dist.py:189-192."""
    for m in model.modules():
        if isinstance(m, (NormDist, NormDistConv)):
            m.p = p


def get_p_norm(model):
    """model/norm_dist.py:194-198."""
    for m in model.modules():
        if isinstance(m, (NormDist, NormDistConv)):
            return m.p
    return None
