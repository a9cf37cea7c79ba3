"""Drop-in for the reference's native module ``norm_dist_cpp``.

The seven functions keep the names, positional order and in-place contract of
the reference binding (model/norm_dist.cpp:22-100): they take torch tensors,
write into caller-allocated tensors and return None.  Each one checks its
arguments like the reference (device, contiguity; a failed check raises
RuntimeError) plus the shape relations the reference leaves unchecked, then
calls the matching C-ABI entry point of libldist_hip.so on the current HIP
stream of the tensors' device.
"""
import torch

from . import _lib


def _check_input(t, name, dtype=torch.float32):
    # reference CHECK_INPUT: is_cuda and is_contiguous (model/norm_dist.cpp:3-5);
    # the dtype test is what data_ptr<float>() enforces there
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")


def _same_device(*ts):
    dev = ts[0].device
    for t in ts[1:]:
        if t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def _expect(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _call(name, device, *args):
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        rc = getattr(_lib.lib(), name)(*args, stream)
    _lib.check(rc, name)


def _p(t):
    return t.data_ptr()


def norm_dist_forward(input, weight, output, G, p):
    """model/norm_dist.cpp:22-28."""
    for t, n in ((input, "input"), (weight, "weight"), (output, "output")):
        _check_input(t, n)
    dev = _same_device(input, weight, output)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _expect(input.dim() == 3 and output.dim() == 3 and weight.dim() == 2, "input/output must be 3-D, weight 2-D")
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(output.size(0) == B and output.size(2) == HW, "output must be (B, CO, HW)")
    _call("ldist_norm_dist_forward", dev, _p(input), _p(weight), B, CO, CI, G, HW, _p(output), float(p))


def norm_dist_backward_input(grad_output, input, weight, output, grad_input, G, p):
    """model/norm_dist.cpp:30-40."""
    for t, n in ((grad_output, "grad_output"), (input, "input"), (weight, "weight"), (output, "output"),
                 (grad_input, "grad_input")):
        _check_input(t, n)
    dev = _same_device(grad_output, input, weight, output, grad_input)
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(tuple(output.shape) == (B, CO, HW) and tuple(grad_output.shape) == (B, CO, HW),
            "output and grad_output must be (B, CO, HW)")
    _expect(tuple(grad_input.shape) == tuple(input.shape) and input.size(0) == B, "grad_input must match input")
    _call("ldist_norm_dist_backward_input", dev, _p(grad_output), _p(input), _p(weight), _p(output), B, CO, CI, G, HW,
          _p(grad_input), float(p))


def norm_dist_backward_weight(grad_output, input, weight, output, grad_weight, G, p):
    """model/norm_dist.cpp:42-52.  grad_weight is accumulated onto (the caller zero-fills it)."""
    for t, n in ((grad_output, "grad_output"), (input, "input"), (weight, "weight"), (output, "output"),
                 (grad_weight, "grad_weight")):
        _check_input(t, n)
    dev = _same_device(grad_output, input, weight, output, grad_weight)
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(tuple(output.shape) == (B, CO, HW) and tuple(grad_output.shape) == (B, CO, HW),
            "output and grad_output must be (B, CO, HW)")
    _expect(tuple(grad_weight.shape) == tuple(weight.shape) and input.size(0) == B, "grad_weight must match weight")
    _call("ldist_norm_dist_backward_weight", dev, _p(grad_output), _p(input), _p(weight), _p(output), B, CO, CI, G,
          HW, _p(grad_weight), float(p))


def norm_dist_backward(grad_output, input, weight, output, grad_input, grad_weight, G, p):
    """Both gradients in one call (the reference's two backward calls, model/norm_dist.cpp:30-52, with every term
    evaluated once where one kernel can serve both).  grad_input is written whole; grad_weight is accumulated onto."""
    for t, n in ((grad_output, "grad_output"), (input, "input"), (weight, "weight"), (output, "output"),
                 (grad_input, "grad_input"), (grad_weight, "grad_weight")):
        _check_input(t, n)
    dev = _same_device(grad_output, input, weight, output, grad_input, grad_weight)
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(tuple(output.shape) == (B, CO, HW) and tuple(grad_output.shape) == (B, CO, HW),
            "output and grad_output must be (B, CO, HW)")
    _expect(tuple(grad_input.shape) == tuple(input.shape), "grad_input must match input")
    _expect(tuple(grad_weight.shape) == tuple(weight.shape) and input.size(0) == B, "grad_weight must match weight")
    _call("ldist_norm_dist_backward", dev, _p(grad_output), _p(input), _p(weight), _p(output), B, CO, CI, G, HW,
          _p(grad_input), _p(grad_weight), float(p))


def inf_dist_forward(input, weight, output, pos, G):
    """model/norm_dist.cpp:54-62."""
    for t, n in ((input, "input"), (weight, "weight"), (output, "output")):
        _check_input(t, n)
    _check_input(pos, "pos", torch.int32)
    dev = _same_device(input, weight, output, pos)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _expect(input.dim() == 3 and weight.dim() == 2, "input must be 3-D, weight 2-D")
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(tuple(output.shape) == (B, CO, HW) and tuple(pos.shape) == (B, CO, HW), "output and pos must be (B, CO, HW)")
    _call("ldist_inf_dist_forward", dev, _p(input), _p(weight), B, CO, CI, G, HW, _p(output), _p(pos))


def inf_dist_forward_values(input, weight, output, G):
    """inf_dist_forward without pos, for a forward pass that no gradient follows (no counterpart in the reference,
    whose forward always computes pos).  Returns False, with nothing written, where the library has no kernel for
    it (anything but a fully connected layer with more than 16 outputs per group and 128-bit loadable rows):
    call inf_dist_forward then."""
    for t, n in ((input, "input"), (weight, "weight"), (output, "output")):
        _check_input(t, n)
    dev = _same_device(input, weight, output)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _expect(input.dim() == 3 and weight.dim() == 2, "input must be 3-D, weight 2-D")
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(tuple(output.shape) == (B, CO, HW), "output must be (B, CO, HW)")
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        rc = _lib.lib().ldist_inf_dist_forward_values(_p(input), _p(weight), B, CO, CI, G, HW, _p(output), stream)
    if rc == _lib.EUNSUPPORTED:
        return False
    _lib.check(rc, "ldist_inf_dist_forward_values")
    return True


def inf_dist_bound_forward(input_lower, input_upper, weight, output_lower, output_upper, G):
    """model/norm_dist.cpp:64-74."""
    for t, n in ((input_lower, "input_lower"), (input_upper, "input_upper"), (weight, "weight"),
                 (output_lower, "output_lower"), (output_upper, "output_upper")):
        _check_input(t, n)
    dev = _same_device(input_lower, input_upper, weight, output_lower, output_upper)
    B, CO, CI, HW = input_lower.size(0), output_lower.size(1), input_lower.size(1), input_lower.size(2)
    _expect(tuple(input_upper.shape) == tuple(input_lower.shape), "input_upper must match input_lower")
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    _expect(tuple(output_lower.shape) == (B, CO, HW) and tuple(output_upper.shape) == (B, CO, HW),
            "outputs must be (B, CO, HW)")
    _call("ldist_inf_dist_bound_forward", dev, _p(input_lower), _p(input_upper), _p(weight), B, CO, CI, G, HW,
          _p(output_lower), _p(output_upper))


def inf_dist_value_bound_forward(input, input_lower, input_upper, weight, output, output_lower, output_upper, G,
                                 mean=None, bias=None):
    """Values and interval bounds in one pass over the weights (no counterpart in model/norm_dist.cpp: the reference
    calls inf_dist_forward and inf_dist_bound_forward one after the other, model/norm_dist.py:134,144-145), with the
    evaluation-mode epilogue (v - mean[c]) + bias[c] per output channel when `mean` / `bias` are given (:146-155)."""
    for t, n in ((input, "input"), (input_lower, "input_lower"), (input_upper, "input_upper"), (weight, "weight"),
                 (output, "output"), (output_lower, "output_lower"), (output_upper, "output_upper")):
        _check_input(t, n)
    tensors = [input, input_lower, input_upper, weight, output, output_lower, output_upper]
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    for t, n in ((mean, "mean"), (bias, "bias")):
        if t is not None:
            _check_input(t, n)
            _expect(tuple(t.shape) == (CO,), f"{n} must be (CO,)")
            tensors.append(t)
    dev = _same_device(*tensors)
    _expect(tuple(input_lower.shape) == tuple(input.shape) and tuple(input_upper.shape) == tuple(input.shape),
            "input_lower and input_upper must match input")
    _expect(weight.size(0) == CO and weight.size(1) * G == CI, "weight must be (CO, CI/G)")
    for t in (output, output_lower, output_upper):
        _expect(tuple(t.shape) == (B, CO, HW), "outputs must be (B, CO, HW)")
    _call("ldist_inf_dist_value_bound_forward", dev, _p(input), _p(input_lower), _p(input_upper), _p(weight), B, CO, CI,
          G, HW, _p(mean) if mean is not None else None, _p(bias) if bias is not None else None, _p(output),
          _p(output_lower), _p(output_upper))


def _inf_backward_input(name, grad_output, pos, grad_input, G):
    _check_input(grad_output, "grad_output")
    _check_input(pos, "pos", torch.int32)
    _check_input(grad_input, "grad_input")
    dev = _same_device(grad_output, pos, grad_input)
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_input.size(2)
    _expect(tuple(pos.shape) == tuple(grad_output.shape), "pos must match grad_output")
    _expect(grad_input.size(0) == B and grad_output.size(2) == HW, "grad_input must be (B, CI, HW)")
    _call(name, dev, _p(grad_output), _p(pos), B, CO, CI, G, HW, _p(grad_input))


def _inf_backward_weight(name, grad_output, pos, grad_weight, G):
    _check_input(grad_output, "grad_output")
    _check_input(pos, "pos", torch.int32)
    _check_input(grad_weight, "grad_weight")
    dev = _same_device(grad_output, pos, grad_weight)
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_weight.size(1) * G, grad_output.size(2)
    _expect(tuple(pos.shape) == tuple(grad_output.shape), "pos must match grad_output")
    _expect(grad_weight.size(0) == CO, "grad_weight must be (CO, CI/G)")
    _call(name, dev, _p(grad_output), _p(pos), B, CO, CI, G, HW, _p(grad_weight))


def inf_dist_backward_input(grad_output, pos, grad_input, G):
    """model/norm_dist.cpp:76-82.  Accumulates onto grad_input (the caller zero-fills it)."""
    _inf_backward_input("ldist_inf_dist_backward_input", grad_output, pos, grad_input, G)


def inf_dist_backward_weight(grad_output, pos, grad_weight, G):
    """model/norm_dist.cpp:84-90.  Accumulates onto grad_weight (the caller zero-fills it)."""
    _inf_backward_weight("ldist_inf_dist_backward_weight", grad_output, pos, grad_weight, G)


# No counterpart in the reference: same results as zero-fill + the two functions above,
# but every element of the gradient is written, so the buffer may be torch.empty.
def inf_dist_backward_input_overwrite(grad_output, pos, grad_input, G):
    _inf_backward_input("ldist_inf_dist_backward_input_overwrite", grad_output, pos, grad_input, G)


def inf_dist_backward_weight_overwrite(grad_output, pos, grad_weight, G):
    _inf_backward_weight("ldist_inf_dist_backward_weight_overwrite", grad_output, pos, grad_weight, G)


def inf_dist_backward_overwrite(grad_output, pos, grad_input, grad_weight, G):
    """Both L_inf gradients in one call, each written whole (what inf_dist_backward_input_overwrite followed by
    inf_dist_backward_weight_overwrite computes): for a fully connected layer the two scatters share one launch."""
    _check_input(grad_output, "grad_output")
    _check_input(pos, "pos", torch.int32)
    _check_input(grad_input, "grad_input")
    _check_input(grad_weight, "grad_weight")
    dev = _same_device(grad_output, pos, grad_input, grad_weight)
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_input.size(2)
    _expect(tuple(pos.shape) == tuple(grad_output.shape), "pos must match grad_output")
    _expect(grad_input.size(0) == B and grad_output.size(2) == HW, "grad_input must be (B, CI, HW)")
    _expect(grad_weight.size(0) == CO and grad_weight.size(1) * G == CI, "grad_weight must be (CO, CI/G)")
    _call("ldist_inf_dist_backward_overwrite", dev, _p(grad_output), _p(pos), B, CO, CI, G, HW, _p(grad_input),
          _p(grad_weight))


def mean_shift(x, y, mean_out=None, running_mean=None, momentum=0.0):
    """y = x minus its per-channel mean over dims 0 and 2 of a (B, C, L) tensor, in one kernel.

    Not in the reference's binding: there the same arithmetic is MeanNorm's torch code
    (model/norm_dist.py:85-96).  ``mean_out`` (C) receives the mean, ``running_mean`` (C) is moved
    by ``momentum`` in place; both are optional.
    """
    _check_input(x, "x")
    _check_input(y, "y")
    _expect(x.dim() == 3 and y.shape == x.shape, "x and y must be (B, C, L) tensors of one shape")
    _expect(y.data_ptr() != x.data_ptr(), "y must not alias x")
    tensors = [x, y]
    for t, n in ((mean_out, "mean_out"), (running_mean, "running_mean")):
        if t is not None:
            _check_input(t, n)
            _expect(t.numel() == x.size(1), f"{n} must have C elements")
            tensors.append(t)
    dev = _same_device(*tensors)
    _call("ldist_mean_shift", dev, _p(x), x.size(0), x.size(1), x.size(2), _p(y),
          None if mean_out is None else _p(mean_out), None if running_mean is None else _p(running_mean),
          float(momentum))


def adamw_lp_step(param, grad, exp_avg, exp_avg_sq, p_norm, lr, beta1, beta2, eps, weight_decay, step):
    """One AdamW step with row-wise l_p weight decay, in place, in one kernel (reference adamw.py:36-85).

    ``param`` is viewed as (param.size(0), rest); ``p_norm`` is None for a module without p, else the
    module's p (float, may be inf).  Not in the reference's binding: there this is torch code.
    """
    tensors = [param, grad, exp_avg, exp_avg_sq]
    for t, n in zip(tensors, ("param", "grad", "exp_avg", "exp_avg_sq")):
        _check_input(t, n)
        _expect(t.shape == param.shape, f"{n} must have the shape of param")
    dev = _same_device(*tensors)
    rows = param.size(0) if param.dim() > 0 else 1
    cols = param.numel() // max(rows, 1)
    _expect(param.numel() > 0, "param must not be empty")
    _call("ldist_adamw_lp_step", dev, _p(param), _p(grad), _p(exp_avg), _p(exp_avg_sq), rows, cols,
          -1.0 if p_norm is None else float(p_norm), float(lr), float(beta1), float(beta2), float(eps),
          float(weight_decay), int(step))


def _conv_args(img, kernel_size, stride, padding, dilation):
    _expect(img.dim() == 4, "img must be (B, C, H, W)")
    B, C, H, W = img.shape
    return B, C, H, W, int(kernel_size), int(kernel_size), int(stride), int(padding), int(dilation)


def conv_output_size(H, W, kernel_size, stride=1, padding=0, dilation=1):
    span = dilation * (kernel_size - 1) + 1
    return (H + 2 * padding - span) // stride + 1, (W + 2 * padding - span) // stride + 1


def unfold(img, cols, kernel_size, stride=1, padding=0, dilation=1):
    """cols (B, C*k*k, HO*WO) = torch.nn.functional.unfold(img, k, dilation, padding, stride), in one kernel."""
    _check_input(img, "img")
    _check_input(cols, "cols")
    dev = _same_device(img, cols)
    B, C, H, W, KH, KW, S, P, D = _conv_args(img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    _expect(cols.shape == (B, C * KH * KW, HO * WO), "cols must be (B, C*k*k, HO*WO)")
    _call("ldist_unfold", dev, _p(img), B, C, H, W, KH, KW, S, P, D, _p(cols))


def fold(grad_cols, grad_img, kernel_size, stride=1, padding=0, dilation=1):
    """grad_img (B, C, H, W) = the adjoint of unfold applied to grad_cols; every element is written."""
    _check_input(grad_cols, "grad_cols")
    _check_input(grad_img, "grad_img")
    dev = _same_device(grad_cols, grad_img)
    B, C, H, W, KH, KW, S, P, D = _conv_args(grad_img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    _expect(grad_cols.shape == (B, C * KH * KW, HO * WO), "grad_cols must be (B, C*k*k, HO*WO)")
    _call("ldist_fold", dev, _p(grad_cols), B, C, H, W, KH, KW, S, P, D, _p(grad_img))


FOLDED_MAX_ROW_FLOATS = 16384   # (C/G) * W must fit the kernel's LDS bins


def inf_dist_backward_input_folded(grad_output, pos, grad_img, G, kernel_size, stride=1, padding=0, dilation=1):
    """Gradient of the L_inf layer with respect to the image: inf_dist_backward_input followed by fold, fused."""
    _check_input(grad_output, "grad_output")
    _check_input(pos, "pos", torch.int32)
    _check_input(grad_img, "grad_img")
    dev = _same_device(grad_output, pos, grad_img)
    B, C, H, W, KH, KW, S, P, D = _conv_args(grad_img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    CO = grad_output.size(1)
    _expect(grad_output.dim() == 3 and grad_output.shape == pos.shape and grad_output.size(0) == B and
            grad_output.size(2) == HO * WO, "grad_output and pos must be (B, CO, HO*WO)")
    _call("ldist_inf_dist_backward_input_folded", dev, _p(grad_output), _p(pos), B, CO, C, G, H, W, KH, KW, S, P, D,
          _p(grad_img))


def inf_dist_conv_forward_supported(C, H, W, CO, G, kernel_size, stride=1, padding=0, dilation=1):
    """True when inf_dist_conv_forward covers the geometry (3x3, dilation 1, stride 1 or 2; a group's channels
    few enough to stay in LDS or a multiple of four; a layer large enough to fill the GPU); otherwise unfold +
    inf_dist_forward is the way."""
    k = int(kernel_size)
    return bool(_lib.lib().ldist_inf_dist_conv_forward_supported(int(C), int(H), int(W), int(CO), int(G), k, k,
                                                                  int(stride), int(padding), int(dilation)))


def inf_dist_conv_forward(img, weight, output, pos, G, kernel_size, stride=1, padding=0, dilation=1):
    """L_inf forward of the conv-shaped layer straight from the image: output, pos (B, CO, HO*WO) equal to
    inf_dist_forward on F.unfold(img, ...), without building the columns."""
    for t, n in ((img, "img"), (weight, "weight"), (output, "output")):
        _check_input(t, n)
    _check_input(pos, "pos", torch.int32)
    dev = _same_device(img, weight, output, pos)
    B, C, H, W, KH, KW, S, P, D = _conv_args(img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    _expect(weight.dim() == 2 and C % G == 0 and weight.size(1) == C // G * KH * KW, "weight must be (CO, C/G*k*k)")
    CO = weight.size(0)
    _expect(output.shape == (B, CO, HO * WO) and pos.shape == output.shape, "output and pos must be (B, CO, HO*WO)")
    _call("ldist_inf_dist_conv_forward", dev, _p(img), _p(weight), B, C, H, W, CO, G, KH, KW, S, P, D, _p(output),
          _p(pos))


def inf_dist_conv_forward_values(img, weight, output, G, kernel_size, stride=1, padding=0, dilation=1):
    """inf_dist_conv_forward without pos, for a forward pass that no gradient follows (no counterpart in the
    reference); the geometries of inf_dist_conv_forward_supported."""
    for t, n in ((img, "img"), (weight, "weight"), (output, "output")):
        _check_input(t, n)
    dev = _same_device(img, weight, output)
    B, C, H, W, KH, KW, S, P, D = _conv_args(img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    _expect(weight.dim() == 2 and C % G == 0 and weight.size(1) == C // G * KH * KW, "weight must be (CO, C/G*k*k)")
    CO = weight.size(0)
    _expect(output.shape == (B, CO, HO * WO), "output must be (B, CO, HO*WO)")
    _call("ldist_inf_dist_conv_forward_values", dev, _p(img), _p(weight), B, C, H, W, CO, G, KH, KW, S, P, D, _p(output))


def norm_dist_conv_supported(C, H, W, CO, G, kernel_size, stride=1, padding=0, dilation=1):
    """True when the three norm_dist_conv_* calls cover the geometry (3x3 windows, more than one output position);
    otherwise unfold + the column calls are the way."""
    k = int(kernel_size)
    return bool(_lib.lib().ldist_norm_dist_conv_supported(int(C), int(H), int(W), int(CO), int(G), k, k, int(stride),
                                                           int(padding), int(dilation)))


def _norm_conv_args(img, weight, output, G, kernel_size, stride, padding, dilation):
    B, C, H, W, KH, KW, S, P, D = _conv_args(img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    _expect(weight.dim() == 2 and C % G == 0 and weight.size(1) == C // G * KH * KW, "weight must be (CO, C/G*k*k)")
    CO = weight.size(0)
    _expect(output.shape == (B, CO, HO * WO), "output must be (B, CO, HO*WO)")
    return B, C, H, W, CO, G, KH, KW, S, P, D


def norm_dist_conv_forward(img, weight, output, G, p, kernel_size, stride=1, padding=0, dilation=1):
    """p-norm forward of the conv-shaped layer straight from the image: output (B, CO, HO*WO) equal to
    norm_dist_forward on F.unfold(img, ...), without building the columns."""
    for t, n in ((img, "img"), (weight, "weight"), (output, "output")):
        _check_input(t, n)
    dev = _same_device(img, weight, output)
    args = _norm_conv_args(img, weight, output, G, kernel_size, stride, padding, dilation)
    _call("ldist_norm_dist_conv_forward", dev, _p(img), _p(weight), *args, _p(output), float(p))


def norm_dist_conv_backward_input(grad_output, img, weight, output, grad_img, G, p, kernel_size, stride=1, padding=0,
                                  dilation=1):
    """Gradient of the p-norm conv-shaped layer with respect to the image: norm_dist_backward_input on the columns
    followed by fold, without either tensor of columns.  Every element of grad_img is written."""
    for t, n in ((grad_output, "grad_output"), (img, "img"), (weight, "weight"), (output, "output"),
                 (grad_img, "grad_img")):
        _check_input(t, n)
    dev = _same_device(grad_output, img, weight, output, grad_img)
    args = _norm_conv_args(img, weight, output, G, kernel_size, stride, padding, dilation)
    _expect(grad_output.shape == output.shape and grad_img.shape == img.shape,
            "grad_output must match output and grad_img the image")
    _call("ldist_norm_dist_conv_backward_input", dev, _p(grad_output), _p(img), _p(weight), _p(output), *args,
          _p(grad_img), float(p))


def norm_dist_conv_backward_weight(grad_output, img, weight, output, grad_weight, G, p, kernel_size, stride=1,
                                   padding=0, dilation=1):
    """Gradient of the p-norm conv-shaped layer with respect to the weight, reading the image instead of the
    columns.  Added onto grad_weight, like norm_dist_backward_weight."""
    for t, n in ((grad_output, "grad_output"), (img, "img"), (weight, "weight"), (output, "output"),
                 (grad_weight, "grad_weight")):
        _check_input(t, n)
    dev = _same_device(grad_output, img, weight, output, grad_weight)
    args = _norm_conv_args(img, weight, output, G, kernel_size, stride, padding, dilation)
    _expect(grad_output.shape == output.shape and grad_weight.shape == weight.shape,
            "grad_output must match output and grad_weight the weight")
    _call("ldist_norm_dist_conv_backward_weight", dev, _p(grad_output), _p(img), _p(weight), _p(output), *args,
          _p(grad_weight), float(p))


def norm_dist_conv_backward(grad_output, img, weight, output, grad_img, grad_weight, G, p, kernel_size, stride=1,
                            padding=0, dilation=1):
    """Both gradients of the p-norm conv-shaped layer from the image in one call (every term evaluated once where
    one kernel can serve both).  grad_img is written whole, grad_weight is added to."""
    for t, n in ((grad_output, "grad_output"), (img, "img"), (weight, "weight"), (output, "output"),
                 (grad_img, "grad_img"), (grad_weight, "grad_weight")):
        _check_input(t, n)
    dev = _same_device(grad_output, img, weight, output, grad_img, grad_weight)
    args = _norm_conv_args(img, weight, output, G, kernel_size, stride, padding, dilation)
    _expect(grad_output.shape == output.shape and grad_img.shape == img.shape and grad_weight.shape == weight.shape,
            "grad_output must match output, grad_img the image and grad_weight the weight")
    _call("ldist_norm_dist_conv_backward", dev, _p(grad_output), _p(img), _p(weight), _p(output), *args, _p(grad_img),
          _p(grad_weight), float(p))


def inf_dist_bound_conv_forward_supported(C, H, W, CO, G, kernel_size, stride=1, padding=0, dilation=1):
    """True when inf_dist_bound_conv_forward covers the geometry (3x3, dilation 1, stride 1 or 2, a layer large
    enough to fill the GPU); otherwise unfold both images and call inf_dist_bound_forward."""
    k = int(kernel_size)
    return bool(_lib.lib().ldist_inf_dist_bound_conv_forward_supported(int(C), int(H), int(W), int(CO), int(G), k, k,
                                                                        int(stride), int(padding), int(dilation)))


def inf_dist_bound_conv_forward(lower_img, upper_img, weight, output_lower, output_upper, G, kernel_size, stride=1,
                                padding=0, dilation=1):
    """Interval bounds of the conv-shaped layer straight from the lower and upper images: equal to
    inf_dist_bound_forward on F.unfold of both, without building the columns."""
    for t, n in ((lower_img, "lower_img"), (upper_img, "upper_img"), (weight, "weight"),
                 (output_lower, "output_lower"), (output_upper, "output_upper")):
        _check_input(t, n)
    dev = _same_device(lower_img, upper_img, weight, output_lower, output_upper)
    _expect(lower_img.shape == upper_img.shape, "lower_img and upper_img must have one shape")
    B, C, H, W, KH, KW, S, P, D = _conv_args(lower_img, kernel_size, stride, padding, dilation)
    HO, WO = conv_output_size(H, W, KH, S, P, D)
    _expect(weight.dim() == 2 and C % G == 0 and weight.size(1) == C // G * KH * KW, "weight must be (CO, C/G*k*k)")
    CO = weight.size(0)
    _expect(output_lower.shape == (B, CO, HO * WO) and output_upper.shape == output_lower.shape,
            "output_lower and output_upper must be (B, CO, HO*WO)")
    _call("ldist_inf_dist_bound_conv_forward", dev, _p(lower_img), _p(upper_img), _p(weight), B, C, H, W, CO, G, KH, KW,
          S, P, D, _p(output_lower), _p(output_upper))


# ---- the compiled PyTorch extension -------------------------------------------------------------------------
# The seven functions of the reference module also exist as a PyTorch-ROCm C++ extension that carries the
# reference's module name, `norm_dist_cpp` (csrc/torch_ext/norm_dist_cpp.cpp: pybind11 over the same C ABI, built by
# `make -C csrc torch_ext` or __graft_entry__.build() into torch_ext/).  Where it has been built, this module hands
# those seven names to it, so the autograd functions of norm_dist.py call a compiled binding as the reference's do;
# the ctypes functions above stay available as `ctypes_binding[name]` and serve every entry point the reference
# module does not have.  Either way the work is done by libldist_hip.so: there is no path without it.
REFERENCE_NAMES = ("norm_dist_forward", "norm_dist_backward_input", "norm_dist_backward_weight", "inf_dist_forward",
                   "inf_dist_bound_forward", "inf_dist_backward_input", "inf_dist_backward_weight")
ctypes_binding = {name: globals()[name] for name in REFERENCE_NAMES}
_extension = None
BINDING = "ctypes"     # or "torch_extension": what the seven reference names are bound to right now


def torch_extension():
    """The compiled module (torch_ext/norm_dist_cpp*.so), or None when it has not been built."""
    global _extension
    if _extension is None:
        import glob
        import importlib.util
        import os
        hits = glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "torch_ext", "norm_dist_cpp*.so"))
        if not hits:
            return None
        _lib.lib()     # libldist_hip.so first: a missing library should be reported by its own message
        spec = importlib.util.spec_from_file_location("norm_dist_cpp", hits[0])
        _extension = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_extension)
    return _extension


def use_torch_extension(on=True):
    """Binds the seven reference names to the compiled extension (on=True; RuntimeError when it has not been built)
    or back to the ctypes functions (on=False).  Returns the binding now in use."""
    global BINDING
    if on:
        ext = torch_extension()
        if ext is None:
            raise RuntimeError("torch_ext/norm_dist_cpp*.so is missing: build it with `make -C csrc torch_ext`")
        for name in REFERENCE_NAMES:
            globals()[name] = getattr(ext, name)
        BINDING = "torch_extension"
    else:
        globals().update(ctypes_binding)
        BINDING = "ctypes"
    return BINDING


try:
    if torch_extension() is not None:
        use_torch_extension(True)
except (RuntimeError, ImportError, OSError):   # no library yet (the first call reports it), or built for another torch
    pass
