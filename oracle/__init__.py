"""CPU oracle for the distance-neuron operators -- TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module.  It is loaded by tests/,
by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``
as the checker the HIP kernels are compared with.

Two restatements live here:

* ``ldist_oracle.c`` (through ctypes): plain-C loops that follow the reference
  kernels' arithmetic (model/inf_dist_cuda.cu, model/norm_dist_cuda.cu).
* ``fallback_norm_dist`` / ``fallback_inf_dist_bound``: the reference's dormant
  pure-torch path (model/norm_dist.py:52-57 and :66-75) restated with batch
  chunking, because the broadcast temporary is B*CO*CI/G*HW floats.  Rows are
  independent, so chunking does not change any result.

All functions take and return CPU float32 / int32 torch tensors shaped like the
reference's: input (B, CI, HW), weight (CO, CI/G), output (B, CO, HW).
"""
import ctypes
import math
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libldist_oracle.so")
_lib = None


def build(force=False):
    """Compile ldist_oracle.c with gcc (about a second)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def num_threads():
    return int(lib().ldist_oracle_num_threads())


def _f(t):
    assert t.dtype == torch.float32 and t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _i(t):
    assert t.dtype == torch.int32 and t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _dims(x, weight, group):
    B, CI, HW = x.shape
    CO = weight.shape[0]
    assert weight.shape[1] * group == CI, "weight.size(1) * group must equal input.size(1)"
    return B, CO, CI, group, HW


def _check(rc, name):
    if rc != 0:
        raise RuntimeError(f"oracle {name} failed with code {rc}")


def inf_dist_forward(x, weight, group=1, literal=False):
    B, CO, CI, G, HW = _dims(x, weight, group)
    out = torch.empty(B, CO, HW, dtype=torch.float32)
    pos = torch.empty(B, CO, HW, dtype=torch.int32)
    fn = lib().ldist_oracle_inf_dist_forward_literal if literal else lib().ldist_oracle_inf_dist_forward
    _check(fn(_f(x), _f(weight), B, CO, CI, G, HW, _f(out), _i(pos)), "inf_dist_forward")
    return out, pos


def inf_dist_bound_forward(lower, upper, weight, group=1):
    B, CO, CI, G, HW = _dims(lower, weight, group)
    assert upper.shape == lower.shape
    out_l = torch.empty(B, CO, HW, dtype=torch.float32)
    out_u = torch.empty(B, CO, HW, dtype=torch.float32)
    _check(lib().ldist_oracle_inf_dist_bound_forward(_f(lower), _f(upper), _f(weight), B, CO, CI, G, HW,
                                                      _f(out_l), _f(out_u)), "inf_dist_bound_forward")
    return out_l, out_u


def inf_dist_backward_input(grad_output, pos, CI, group=1, grad_input=None):
    B, CO, HW = grad_output.shape
    if grad_input is None:
        grad_input = torch.zeros(B, CI, HW, dtype=torch.float32)
    _check(lib().ldist_oracle_inf_dist_backward_input(_f(grad_output), _i(pos), B, CO, CI, group, HW,
                                                       _f(grad_input)), "inf_dist_backward_input")
    return grad_input


def inf_dist_backward_weight(grad_output, pos, CI, group=1, grad_weight=None):
    B, CO, HW = grad_output.shape
    if grad_weight is None:
        grad_weight = torch.zeros(CO, CI // group, dtype=torch.float32)
    _check(lib().ldist_oracle_inf_dist_backward_weight(_f(grad_output), _i(pos), B, CO, CI, group, HW,
                                                        _f(grad_weight)), "inf_dist_backward_weight")
    return grad_weight


def inf_dist_backward_input_f64(grad_output, pos, CI, group=1):
    """The same scatter as inf_dist_backward_input (reference model/inf_dist_cuda.cu:143-156) with the sums left in
    float64 -- the exact column gradient, for checks that go on summing it (fold) before anything is rounded.
    torch.scatter_add_ along k; indices past K are dropped like the C loop drops them."""
    B, CO, HW = grad_output.shape
    K, NG = CI // group, CO // group
    idx = (pos & 0x7FFFFFFF).long().reshape(B, group, NG, HW)
    g = grad_output.double().reshape(B, group, NG, HW)
    sg = torch.where(pos.reshape(B, group, NG, HW) >= 0, g, -g)
    keep = idx < K
    acc = torch.zeros(B, group, K, HW, dtype=torch.float64)
    acc.scatter_add_(2, torch.where(keep, idx, torch.zeros_like(idx)), torch.where(keep, sg, torch.zeros_like(sg)))
    return acc.reshape(B, CI, HW)


def norm_dist_forward(x, weight, group, p, f32_reference_order=False):
    B, CO, CI, G, HW = _dims(x, weight, group)
    out = torch.empty(B, CO, HW, dtype=torch.float32)
    fn = lib().ldist_oracle_norm_dist_forward_f32 if f32_reference_order else lib().ldist_oracle_norm_dist_forward
    _check(fn(_f(x), _f(weight), B, CO, CI, G, HW, _f(out), ctypes.c_float(p)), "norm_dist_forward")
    return out


def norm_dist_backward_input(grad_output, x, weight, output, group, p, with_abs_terms=False):
    """with_abs_terms=True also returns sum_n |term| per element (the rounding-error scale)."""
    B, CO, CI, G, HW = _dims(x, weight, group)
    grad_input = torch.empty_like(x)
    mag = torch.empty_like(x) if with_abs_terms else None
    _check(lib().ldist_oracle_norm_dist_backward_input(_f(grad_output), _f(x), _f(weight), _f(output), B, CO, CI, G,
                                                        HW, _f(grad_input), ctypes.c_float(p),
                                                        _f(mag) if with_abs_terms else None),
           "norm_dist_backward_input")
    return (grad_input, mag) if with_abs_terms else grad_input


def norm_dist_backward_weight(grad_output, x, weight, output, group, p, grad_weight=None, with_abs_terms=False):
    B, CO, CI, G, HW = _dims(x, weight, group)
    if grad_weight is None:
        grad_weight = torch.zeros_like(weight)
    mag = torch.empty_like(weight) if with_abs_terms else None
    _check(lib().ldist_oracle_norm_dist_backward_weight(_f(grad_output), _f(x), _f(weight), _f(output), B, CO, CI, G,
                                                         HW, _f(grad_weight), ctypes.c_float(p),
                                                         _f(mag) if with_abs_terms else None),
           "norm_dist_backward_weight")
    return (grad_weight, mag) if with_abs_terms else grad_weight


# --------------------------------------------------------------------------- #
# The reference's pure-torch path, restated (model/norm_dist.py:52-57, 66-75). #
# --------------------------------------------------------------------------- #
def _chunk_rows(B, per_row_floats, budget_floats=1 << 26):
    return max(1, min(B, budget_floats // max(1, per_row_floats)))


def fallback_norm_dist(x, weight, group, p, rows_per_chunk=None):
    """y = norm(d / n, p) * n with n = norm(d, inf), d the broadcast difference
    (model/norm_dist.py:53-57).  Differentiable like the reference's."""
    B, CI, HW = x.shape
    CO = weight.shape[0]
    step = rows_per_chunk or _chunk_rows(B, CO * (CI // group) * HW)
    outs = []
    for s in range(0, B, step):
        xs = x[s:s + step]
        y = xs.reshape(xs.size(0), group, 1, -1, HW) - weight.view(group, -1, weight.size(-1), 1)
        with torch.no_grad():
            normalize = torch.norm(y, dim=3, p=float("inf"), keepdim=True)
        y = torch.norm(y / normalize, dim=3, p=p, keepdim=True) * normalize
        outs.append(y.reshape(y.size(0), -1, y.size(-1)))
    return torch.cat(outs, dim=0)


def fallback_inf_dist_bound(lower, upper, weight, group, rows_per_chunk=None):
    """model/norm_dist.py:66-75."""
    B, CI, HW = lower.shape
    CO = weight.shape[0]
    step = rows_per_chunk or _chunk_rows(B, 4 * CO * (CI // group) * HW)
    w = weight.view(group, -1, weight.size(-1), 1)
    lo, up = [], []
    for s in range(0, B, step):
        xl, xu = lower[s:s + step], upper[s:s + step]
        shape = xl.size(0), CO, HW
        y1 = xl.reshape(xl.size(0), group, 1, -1, HW) - w
        y2 = xu.reshape(xu.size(0), group, 1, -1, HW) - w
        a1, a2 = y1.abs(), y2.abs()
        up.append(torch.maximum(a1, a2).max(dim=3)[0].reshape(shape))
        ol = torch.minimum(a1, a2)
        ol[(y1 < 0) & (y2 > 0)] = 0
        lo.append(ol.max(dim=3)[0].reshape(shape))
    return torch.cat(lo, dim=0), torch.cat(up, dim=0)


def fallback_inf_dist_values(x, weight, group, rows_per_chunk=None):
    """max_k |x - w| by broadcasting; what fallback_norm_dist reduces to at p = inf
    without the 0/0 it produces when a row's maximum is zero."""
    B, CI, HW = x.shape
    CO = weight.shape[0]
    step = rows_per_chunk or _chunk_rows(B, CO * (CI // group) * HW)
    outs = []
    for s in range(0, B, step):
        xs = x[s:s + step]
        y = xs.reshape(xs.size(0), group, 1, -1, HW) - weight.view(group, -1, weight.size(-1), 1)
        outs.append(y.abs().max(dim=3)[0].reshape(xs.size(0), CO, HW))
    return torch.cat(outs, dim=0)


def is_inf(p):
    return math.isinf(p)


def mean_shift(x, running_mean=None, momentum=0.1):
    """(y, mean) of the per-channel mean shift of a (B, C, L) tensor; moves running_mean in place if given."""
    B, C, L = x.shape
    y = torch.empty_like(x)
    mean = torch.empty(C, dtype=torch.float32)
    _check(lib().ldist_oracle_mean_shift(_f(x), B, C, L, _f(y), _f(mean),
                                         None if running_mean is None else _f(running_mean),
                                         ctypes.c_float(momentum)), "mean_shift")
    return y, mean


def adamw_lp_step(param, grad, exp_avg, exp_avg_sq, p_norm, lr, betas, eps, weight_decay, step):
    """In place on param (2-D view rows x cols), exp_avg, exp_avg_sq.  p_norm None = the module has no p."""
    rows = param.size(0)
    cols = param.numel() // rows
    pn = -1.0 if p_norm is None else float(p_norm)
    _check(lib().ldist_oracle_adamw_lp_step(_f(param), None if grad is None else _f(grad),
                                            None if exp_avg is None else _f(exp_avg),
                                            None if exp_avg_sq is None else _f(exp_avg_sq), rows, cols,
                                            ctypes.c_double(pn), ctypes.c_double(lr), ctypes.c_double(betas[0]),
                                            ctypes.c_double(betas[1]), ctypes.c_double(eps),
                                            ctypes.c_double(weight_decay), int(step)), "adamw_lp_step")
