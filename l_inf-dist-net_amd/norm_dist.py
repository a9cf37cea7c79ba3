"""Distance-neuron operators and layers with the reference's Python interface.

Public names, signatures and return conventions follow the reference's
model/norm_dist.py so that its callers work unchanged:

    DistF                      autograd function            (reference :7-47)
    norm_dist, inf_dist_bound  functional API               (reference :49-76)
    MeanNorm                   per-channel mean shift       (reference :78-100)
    NormDistConv, NormDist     conv / fully connected layer (reference :102-187)
    set_p_norm, get_p_norm     p of every layer of a model  (reference :189-198)

The native calls go through ``norm_dist_cpp`` (this package's ctypes binding of
libldist_hip.so).  Not in the reference: ``MeanNormDist`` and the keyword
spellings ``groups`` / ``mean_shift`` accepted by the layers.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import norm_dist_cpp

_INF = float("inf")
def _out_shape(x, weight):
    return x.size(0), weight.size(0), x.size(2)


class DistF(torch.autograd.Function):
    """y[b, n, hw] = || x[b, group(n), :, hw] - weight[n, :] ||_p for p = inf or p > 1.

    x is (B, CI, HW), weight (CO, CI/group).  At p = inf the forward also records
    which input attains the maximum; the backward routes the gradient there.
    """

    @staticmethod
    def forward(ctx, x, weight, group, p, tag):
        assert weight.size(1) * group == x.size(1)
        if not (math.isinf(p) or p > 1):
            raise NotImplementedError
        y = torch.empty(_out_shape(x, weight), device=x.device, dtype=x.dtype)
        if math.isinf(p):
            argmax = torch.empty(y.shape, device=x.device, dtype=torch.int32)
            norm_dist_cpp.inf_dist_forward(x, weight, y, argmax, group)
            ctx.save_for_backward(x, weight, y, argmax)
        else:
            norm_dist_cpp.norm_dist_forward(x, weight, y, group, p)
            ctx.save_for_backward(x, weight, y)
        ctx.group, ctx.p, ctx.tag = group, p, tag
        return y

    @staticmethod
    def backward(ctx, grad_output):
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        g = grad_output.contiguous()
        gx = gw = None
        if math.isinf(ctx.p):
            x, weight, _, argmax = ctx.saved_tensors
            # the scatter kernels write every element, zeros included: no fill needed here
            if want_x and want_w:   # one call: a fully connected layer's two scatters share a launch
                gx, gw = torch.empty_like(x), torch.empty_like(weight)
                norm_dist_cpp.inf_dist_backward_overwrite(g, argmax, gx, gw, ctx.group)
            elif want_x:
                gx = torch.empty_like(x)
                norm_dist_cpp.inf_dist_backward_input_overwrite(g, argmax, gx, ctx.group)
            elif want_w:
                gw = torch.empty_like(weight)
                norm_dist_cpp.inf_dist_backward_weight_overwrite(g, argmax, gw, ctx.group)
        else:
            x, weight, y = ctx.saved_tensors
            if want_x and want_w:
                # every term belongs to both sums: one call, which evaluates it once where one kernel can serve both
                gx, gw = torch.empty_like(x), torch.zeros_like(weight)
                norm_dist_cpp.norm_dist_backward(g, x, weight, y, gx, gw, ctx.group, ctx.p)
            else:
                if want_x:
                    gx = torch.empty_like(x)
                    norm_dist_cpp.norm_dist_backward_input(g, x, weight, y, gx, ctx.group, ctx.p)
                if want_w:
                    gw = torch.zeros_like(weight)  # this kernel adds onto the buffer
                    norm_dist_cpp.norm_dist_backward_weight(g, x, weight, y, gw, ctx.group, ctx.p)
        return gx, gw, None, None, None


class _Unfold(torch.autograd.Function):
    """F.unfold for float32 GPU images as one native kernel, with the native fold as its backward."""

    @staticmethod
    def forward(ctx, img, kernel_size, dilation, padding, stride):
        img = img.contiguous()
        ho, wo = norm_dist_cpp.conv_output_size(img.size(2), img.size(3), kernel_size, stride, padding, dilation)
        cols = torch.empty(img.size(0), img.size(1) * kernel_size * kernel_size, ho * wo, device=img.device,
                           dtype=img.dtype)
        norm_dist_cpp.unfold(img, cols, kernel_size, stride, padding, dilation)
        ctx.geometry = (img.shape, kernel_size, stride, padding, dilation)
        return cols

    @staticmethod
    def backward(ctx, grad_cols):
        shape, kernel_size, stride, padding, dilation = ctx.geometry
        grad_img = torch.empty(shape, device=grad_cols.device, dtype=grad_cols.dtype)
        norm_dist_cpp.fold(grad_cols.contiguous(), grad_img, kernel_size, stride, padding, dilation)
        return grad_img, None, None, None, None


class _ConvInfDist(torch.autograd.Function):
    """The L_inf layer on an image.  Forward: the kernel that reads the image directly where it covers the
    geometry, else unfold + distance forward.  Backward: the gradient with respect to the image directly
    (scatter and fold fused), so the nine times larger gradient of the columns never exists.  Same results
    as unfold + DistF."""

    @staticmethod
    def forward(ctx, img, weight, group, kernel_size, dilation, padding, stride):
        if norm_dist_cpp.inf_dist_conv_forward_supported(img.size(1), img.size(2), img.size(3), weight.size(0), group,
                                                         kernel_size, stride, padding, dilation):
            img = img.contiguous()
            ho, wo = norm_dist_cpp.conv_output_size(img.size(2), img.size(3), kernel_size, stride, padding, dilation)
            y = torch.empty(img.size(0), weight.size(0), ho * wo, device=img.device, dtype=img.dtype)
            argmax = torch.empty(y.shape, device=img.device, dtype=torch.int32)
            norm_dist_cpp.inf_dist_conv_forward(img, weight, y, argmax, group, kernel_size, stride, padding, dilation)
            ctx.geometry = (img.shape, kernel_size, stride, padding, dilation)
        else:
            cols = _Unfold.forward(ctx, img, kernel_size, dilation, padding, stride)
            y = torch.empty(_out_shape(cols, weight), device=img.device, dtype=img.dtype)
            argmax = torch.empty(y.shape, device=img.device, dtype=torch.int32)
            norm_dist_cpp.inf_dist_forward(cols, weight, y, argmax, group)
        ctx.save_for_backward(argmax)
        ctx.group, ctx.weight_shape = group, weight.shape
        return y

    @staticmethod
    def backward(ctx, grad_output):
        (argmax,) = ctx.saved_tensors
        shape, kernel_size, stride, padding, dilation = ctx.geometry
        g = grad_output.contiguous()
        grad_img = grad_w = None
        if ctx.needs_input_grad[0]:
            grad_img = torch.empty(shape, device=g.device, dtype=g.dtype)
            norm_dist_cpp.inf_dist_backward_input_folded(g, argmax, grad_img, ctx.group, kernel_size, stride, padding,
                                                         dilation)
        if ctx.needs_input_grad[1]:
            grad_w = torch.empty(ctx.weight_shape, device=g.device, dtype=g.dtype)
            norm_dist_cpp.inf_dist_backward_weight_overwrite(g, argmax, grad_w, ctx.group)
        return grad_img, grad_w, None, None, None, None, None


class _ConvNormDist(torch.autograd.Function):
    """The p-norm layer (finite p) on an image, forward and both gradients from the image itself: neither the
    unfolded input nor the gradient of the columns exists.  Same results as unfold + DistF to float rounding."""

    @staticmethod
    def forward(ctx, img, weight, group, p, kernel_size, dilation, padding, stride):
        img = img.contiguous()
        weight = weight.contiguous()
        ho, wo = norm_dist_cpp.conv_output_size(img.size(2), img.size(3), kernel_size, stride, padding, dilation)
        y = torch.empty(img.size(0), weight.size(0), ho * wo, device=img.device, dtype=img.dtype)
        norm_dist_cpp.norm_dist_conv_forward(img, weight, y, group, p, kernel_size, stride, padding, dilation)
        ctx.save_for_backward(img, weight, y)
        ctx.group, ctx.p, ctx.window = group, p, (kernel_size, stride, padding, dilation)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        img, weight, y = ctx.saved_tensors
        g = grad_output.contiguous()
        grad_img = grad_w = None
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[1]:   # every term belongs to both sums: one call
            grad_img, grad_w = torch.empty_like(img), torch.zeros_like(weight)
            norm_dist_cpp.norm_dist_conv_backward(g, img, weight, y, grad_img, grad_w, ctx.group, ctx.p, *ctx.window)
        elif ctx.needs_input_grad[0]:
            grad_img = torch.empty_like(img)   # the call writes every element
            norm_dist_cpp.norm_dist_conv_backward_input(g, img, weight, y, grad_img, ctx.group, ctx.p, *ctx.window)
        elif ctx.needs_input_grad[1]:
            grad_w = torch.zeros_like(weight)  # this kernel adds onto the buffer
            norm_dist_cpp.norm_dist_conv_backward_weight(g, img, weight, y, grad_w, ctx.group, ctx.p, *ctx.window)
        return grad_img, grad_w, None, None, None, None, None, None


def _pairwise_difference(inp, weight, group):
    """(B, G, CO/G, CI/G, HW) tensor of input minus weight, by broadcasting."""
    b, _, hw = inp.shape
    return inp.view(b, group, 1, -1, hw) - weight.view(group, -1, weight.size(-1), 1)


def norm_dist(input, weight, group, p, use_custom_cuda_func=True, tag=None):
    """Distances between every input column and every weight row.

    use_custom_cuda_func=False evaluates the same quantity with dense torch ops
    (the broadcast difference is B*CO*CI/group*HW floats), as the reference's
    option of that name does; it is never chosen automatically.
    """
    if use_custom_cuda_func:
        # No gradient will follow (evaluation, torch.no_grad(), the value path of a certification pass): the argmax
        # that the reference always computes (model/norm_dist.py:14-15) has no reader, and the kernel without it is
        # faster.  Where the library has no such kernel for the layout the call says so and the usual path runs.
        if math.isinf(p) and not (torch.is_grad_enabled() and (input.requires_grad or weight.requires_grad)):
            assert weight.size(1) * group == input.size(1)
            y = torch.empty(_out_shape(input, weight), device=input.device, dtype=input.dtype)
            if norm_dist_cpp.inf_dist_forward_values(input, weight, y, group):
                return y
        return DistF.apply(input, weight, group, p, tag)
    diff = _pairwise_difference(input, weight, group)
    with torch.no_grad():
        scale = torch.norm(diff, dim=3, p=_INF, keepdim=True)
    dist = torch.norm(diff / scale, dim=3, p=p, keepdim=True) * scale
    return dist.view(dist.size(0), -1, dist.size(-1))


def inf_dist_bound(input_lower, input_upper, weight, group, use_custom_cuda_func=True, tag=None):
    """Interval bounds of the L_inf distance for inputs in [input_lower, input_upper].

    Returns (output_lower, output_upper); neither carries gradient.
    """
    shape = _out_shape(input_lower, weight)
    if use_custom_cuda_func:
        lo = input_lower.new_empty(shape)
        hi = input_upper.new_empty(shape)
        norm_dist_cpp.inf_dist_bound_forward(input_lower, input_upper, weight, lo, hi, group)
        return lo, hi
    d_lo = _pairwise_difference(input_lower, weight, group)
    d_hi = _pairwise_difference(input_upper, weight, group)
    a_lo, a_hi = d_lo.abs(), d_hi.abs()
    hi = torch.maximum(a_lo, a_hi).amax(dim=3).view(shape)
    straddles = (d_lo < 0) & (d_hi > 0)          # the weight lies strictly inside the interval
    nearest = torch.where(straddles, torch.zeros_like(a_lo), torch.minimum(a_lo, a_hi))
    return nearest.amax(dim=3).view(shape), hi


def _channel_mean(flat):
    # the reference's expression (model/norm_dist.py:88-91)
    return flat.mean(dim=-1).mean(dim=0) if flat.size(-1) > 1 else flat.squeeze(-1).mean(dim=0)


def _native_shift(flat):
    return flat.is_cuda and flat.dtype == torch.float32


class _BatchMeanShift(torch.autograd.Function):
    """flat (B, C, L) minus its per-channel mean over B and L; moves owner.running_mean.

    float32 CUDA tensors go through one native kernel per direction (``norm_dist_cpp.mean_shift``);
    the reference's torch expressions (model/norm_dist.py:87-96) cost five small kernels per layer
    forward and, through autograd, as many backward.  Other tensors take those torch expressions,
    with the backward gx = gy - mean(gy) written out.
    """

    @staticmethod
    def forward(ctx, flat, owner):
        ctx.set_materialize_grads(False)
        if _native_shift(flat):
            flat = flat.contiguous()
            shifted = torch.empty_like(flat)
            norm_dist_cpp.mean_shift(flat, shifted, None, owner.running_mean, owner.momentum)
            return shifted
        mean = _channel_mean(flat)
        owner.running_mean.mul_(1 - owner.momentum).add_(mean, alpha=owner.momentum)
        return flat - mean.unsqueeze(-1)

    @staticmethod
    def backward(ctx, grad_y):
        if grad_y is None:
            return None, None
        if _native_shift(grad_y):
            grad_y = grad_y.contiguous()
            grad_x = torch.empty_like(grad_y)
            norm_dist_cpp.mean_shift(grad_y, grad_x)
            return grad_x, None
        return grad_y - _channel_mean(grad_y).unsqueeze(-1), None


class MeanNorm(nn.Module):
    """Subtracts a per-channel mean: the batch mean in training mode (which also moves
    ``running_mean`` by ``momentum``), ``running_mean`` in eval mode."""

    def __init__(self, out_channels, momentum=0.1):
        super().__init__()
        self.out_channels = out_channels
        self.momentum = momentum
        self.register_buffer("running_mean", torch.zeros(out_channels))

    def forward(self, x):
        flat = x.view(x.size(0), x.size(1), -1)
        if self.training:
            return _BatchMeanShift.apply(flat, self).view_as(x)
        return (flat - self.running_mean.unsqueeze(-1)).view_as(x)

    def extra_repr(self):
        return str(self.out_channels)


class NormDistConv(nn.Module):
    """Convolution-shaped layer of distance neurons.

    forward(x, lower=None, upper=None) -> (y, lower', upper').  Interval bounds are
    propagated only at p = inf in eval mode.  ``p`` starts at 0 and has to be set
    (``set_p_norm``) before the first forward.
    """

    tag = 0

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, group=1, p=0,
                 bias=True, mean_normalize=False, identity_init=True, groups=None, mean_shift=None):
        super().__init__()
        group = group if groups is None else groups
        mean_normalize = mean_normalize if mean_shift is None else mean_shift
        assert in_channels % group == 0
        assert out_channels % group == 0
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride, self.padding, self.dilation = kernel_size, stride, padding, dilation
        self.group = group
        self.p = p

        per_group = in_channels // group
        w = torch.randn(out_channels, per_group, kernel_size, kernel_size)
        if identity_init and in_channels <= out_channels:
            rows = torch.arange(out_channels)
            centre = kernel_size // 2
            w[rows, rows % per_group, centre, centre] = -10.0
        self.weight = nn.Parameter(w)
        self.normalize = MeanNorm(out_channels) if mean_normalize else None
        self.bias = nn.Parameter(torch.zeros(out_channels)) if bias else None

        NormDistConv.tag += 1
        self.tag = NormDistConv.tag

    def _columns(self, t):
        """(B, C*k*k, L) patches of t; a 1x1 window needs no unfold (which launches one kernel per image)."""
        if self.kernel_size == 1 and self.stride == 1 and self.padding == 0:
            return t.reshape(t.size(0), t.size(1), -1).contiguous()   # F.unfold always hands over a contiguous tensor
        if t.is_cuda and t.dtype == torch.float32:
            return _Unfold.apply(t, self.kernel_size, self.dilation, self.padding, self.stride)
        return F.unfold(t, self.kernel_size, self.dilation, self.padding, self.stride)

    def _fused_inf_conv(self, x):
        """True when the image-space L_inf path applies: a real window, p = inf, float32 on the GPU, and one
        image row of a group small enough for the fused backward kernel."""
        return (math.isinf(self.p) and x.is_cuda and x.dtype == torch.float32 and
                not (self.kernel_size == 1 and self.stride == 1 and self.padding == 0) and
                (self.in_channels // self.group) * x.size(3) <= norm_dist_cpp.FOLDED_MAX_ROW_FLOATS)

    # Finite p: "image" runs the layer from the image (nothing of the unfolded size is allocated); "columns" runs native
    # unfold + the column kernels + native fold, which takes about as long (within 5 % either way on the reference's
    # conv nets) and holds two tensors of nine times the image's size while it runs.  Not in the reference, which
    # always unfolds.
    finite_p_route = "image"

    def _norm_from_image(self, x):
        """True when the p-norm layer runs from the image (finite p, float32 on the GPU, a geometry the image
        kernels cover, and `finite_p_route` says so)."""
        return (self.finite_p_route == "image" and
                not math.isinf(self.p) and self.p > 1 and x.is_cuda and x.dtype == torch.float32 and
                self.weight.dtype == torch.float32 and
                norm_dist_cpp.norm_dist_conv_supported(self.in_channels, x.size(2), x.size(3), self.out_channels,
                                                       self.group, self.kernel_size, self.stride, self.padding,
                                                       self.dilation))

    def _bound_from_images(self, lower, upper):
        """True when the interval bounds can be computed straight from the two images (the bound path carries no
        gradient, as in the reference: it runs in evaluation mode only)."""
        return (lower.is_cuda and lower.dtype == torch.float32 and upper.dtype == torch.float32 and
                not (self.kernel_size == 1 and self.stride == 1 and self.padding == 0) and
                norm_dist_cpp.inf_dist_bound_conv_forward_supported(self.in_channels, lower.size(2), lower.size(3),
                                                                    self.out_channels, self.group, self.kernel_size,
                                                                    self.stride, self.padding, self.dilation))

    def _shift(self, t):
        if self.normalize is not None:
            t = self.normalize(t)
        if self.bias is not None:
            t = t + self.bias.view(1, -1, 1, 1)
        return t

    # Outputs per group up to which the one-pass kernel for values and bounds beats the two separate kernels (the
    # head of the 5120-wide net at batch 1024: 31 us against 24 + 28 us and six elementwise shifts).  For wide layers
    # it is slower: one pass holds three accumulator sets and cannot pair the values in one v_max3 (4.6 ms against
    # 1.25 + 2.67 ms on 1024 x 5120 -> 5120).
    FUSED_VALUE_BOUND_MAX_OUTPUTS = 16

    def _value_and_bounds_in_one_pass(self, x, lower, upper):
        """True when values and bounds of this layer come from one kernel call: no gradient is wanted, the layer has
        no window (fc layers and 1x1 convolutions) and few outputs per group (see FUSED_VALUE_BOUND_MAX_OUTPUTS)."""
        return (x.is_cuda and all(t.dtype == torch.float32 for t in (x, lower, upper, self.weight)) and
                not torch.is_grad_enabled() and math.isinf(self.p) and not self.training and
                self.kernel_size == 1 and self.stride == 1 and self.padding == 0 and   # windows: the image kernels
                self.out_channels // self.group <= self.FUSED_VALUE_BOUND_MAX_OUTPUTS)

    # Which kernels the last forward call took, e.g. {"values": "image", "bounds": None}: "image" (straight from
    # the (B, C, H, W) tensor), "columns" (patches first: the reference's only route, and where every window the image
    # kernels do not cover ends up), "one_pass" (values and bounds from one kernel).  Not in the reference.
    last_route = None

    def forward(self, x, lower=None, upper=None):
        span = self.kernel_size - 2 * self.padding
        out_hw = ((x.size(2) - span) // self.stride + 1, (x.size(3) - span) // self.stride + 1)
        w2d = self.weight.view(self.weight.size(0), -1)
        if lower is not None and upper is not None and self._value_and_bounds_in_one_pass(x, lower, upper):
            self.last_route = {"values": "one_pass", "bounds": "one_pass"}
            cx, cl, cu = (self._columns(t).contiguous() for t in (x, lower, upper))
            y = torch.empty(x.size(0), w2d.size(0), out_hw[0] * out_hw[1], device=x.device, dtype=x.dtype)
            lo, hi = torch.empty_like(y), torch.empty_like(y)
            norm_dist_cpp.inf_dist_value_bound_forward(
                cx, cl, cu, w2d.detach().contiguous(), y, lo, hi, self.group,
                None if self.normalize is None else self.normalize.running_mean,
                None if self.bias is None else self.bias.detach())
            shape = (x.size(0), -1, *out_hw)
            return y.view(shape), lo.view(shape), hi.view(shape)
        route = {"values": "columns", "bounds": None}
        if self._fused_inf_conv(x):
            wants_grad = torch.is_grad_enabled() and (x.requires_grad or w2d.requires_grad)
            from_image = norm_dist_cpp.inf_dist_conv_forward_supported(
                x.size(1), x.size(2), x.size(3), w2d.size(0), self.group, self.kernel_size, self.stride, self.padding,
                self.dilation)
            route["values"] = "image" if from_image else "columns"   # _ConvInfDist decides by the same call
            if wants_grad or not from_image:
                y = _ConvInfDist.apply(x, w2d, self.group, self.kernel_size, self.dilation, self.padding, self.stride)
            else:   # no gradient follows: the argmax has no reader, and the kernel without it is faster
                ho, wo = out_hw
                y = torch.empty(x.size(0), w2d.size(0), ho * wo, device=x.device, dtype=x.dtype)
                norm_dist_cpp.inf_dist_conv_forward_values(x.contiguous(), w2d, y, self.group, self.kernel_size,
                                                           self.stride, self.padding, self.dilation)
        elif self._norm_from_image(x):
            route["values"] = "image"
            y = _ConvNormDist.apply(x, w2d, self.group, self.p, self.kernel_size, self.dilation, self.padding,
                                    self.stride)
        else:
            y = norm_dist(self._columns(x), w2d, self.group, p=self.p, tag=self.tag)
        y = self._shift(y.view(x.size(0), -1, *out_hw))  # in training mode only y moves the running mean
        self.last_route = route
        if lower is None or upper is None:
            return y, None, None
        assert math.isinf(self.p) and not self.training
        route["bounds"] = "columns"
        if self._bound_from_images(lower, upper):
            route["bounds"] = "image"
            lo = torch.empty(x.size(0), w2d.size(0), out_hw[0] * out_hw[1], device=x.device, dtype=x.dtype)
            hi = torch.empty_like(lo)
            with torch.no_grad():
                norm_dist_cpp.inf_dist_bound_conv_forward(lower.contiguous(), upper.contiguous(), w2d.detach(), lo, hi,
                                                          self.group, self.kernel_size, self.stride, self.padding,
                                                          self.dilation)
            return y, self._shift(lo.view_as(y)), self._shift(hi.view_as(y))
        lo, hi = inf_dist_bound(self._columns(lower), self._columns(upper), w2d, self.group, tag=self.tag)
        return y, self._shift(lo.view_as(y)), self._shift(hi.view_as(y))

    def extra_repr(self):
        parts = [f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, stride={self.stride}"]
        if self.padding != 0:
            parts.append(f"padding={self.padding}")
        if self.dilation != 1:
            parts.append(f"dilation={self.dilation}")
        if self.group != 1:
            parts.append(f"group={self.group}")
        if self.bias is None:
            parts.append("bias=False")
        return ", ".join(parts)


class NormDist(NormDistConv):
    """Fully connected layer of distance neurons: a 1x1 NormDistConv applied to (B, C, 1, 1)."""

    def __init__(self, in_features, out_features, p=0, bias=True, mean_normalize=False, identity_init=True,
                 mean_shift=None):
        super().__init__(in_features, out_features, 1, p=p, bias=bias, mean_normalize=mean_normalize,
                         identity_init=identity_init, mean_shift=mean_shift)

    def forward(self, x, lower=None, upper=None):
        as_image = lambda t: None if t is None else t.reshape(t.size(0), t.size(1), 1, 1)
        outs = super().forward(as_image(x), as_image(lower), as_image(upper))
        return tuple(None if t is None else t.reshape(t.size(0), t.size(1)) for t in outs)

    def extra_repr(self):
        return f"in_features={self.in_channels}, out_features={self.out_channels}, bias={self.bias is not None}"


class MeanNormDist(NormDist):
    """NormDist with the mean shift switched on and no bias (no class of this name in the reference)."""

    def __init__(self, in_features, out_features, p=0, bias=False, identity_init=True):
        super().__init__(in_features, out_features, p=p, bias=bias, mean_normalize=True, identity_init=identity_init)


def _dist_layers(model):
    return (m for m in model.modules() if isinstance(m, NormDistConv))  # NormDist is a subclass


def set_p_norm(model, p):
    for layer in _dist_layers(model):
        layer.p = p


def get_p_norm(model):
    for layer in _dist_layers(model):
        return layer.p
    return None
