"""AdamW with the reference's row-wise l_p weight decay (reference adamw.py:6-87).

The decay pulls every row w of a parameter (first dimension = rows, the rest flattened)
along the gradient of ||w||_p^2 / 2, with p the current p of the module that owns the
parameter:  w_i -= lr*wd * (|w_i| / ||w||_p)^(p-2) * w_i.  For p = inf only the entry of
largest magnitude in a row decays; a module without p gets plain multiplicative decay;
a bias (rows of one element) therefore decays elementwise.  The Adam update follows on
the decayed parameter.

float32 CUDA parameters take the whole step in one native kernel per tensor
(``norm_dist_cpp.adamw_lp_step``); the reference runs about sixteen elementwise torch
kernels per tensor.  Anything else (CPU tensors, other dtypes, non-contiguous
parameters) goes through the torch expressions below, which spell out the same arithmetic.
"""
import math

import torch
from torch.optim import Optimizer

from . import norm_dist_cpp
from .norm_dist import get_p_norm


def lp_weight_decay_(param, p_norm, lr, weight_decay, eps):
    """The decay part alone, in place, with torch ops (reference adamw.py:40-56)."""
    scale = lr * weight_decay
    if p_norm is None:
        param.mul_(1 - scale)
        return param
    rows = param.view(param.size(0), -1) if param.dim() > 0 else param.view(1, 1)
    if math.isinf(p_norm):
        top = rows.abs().argmax(dim=1, keepdim=True)
        rows.scatter_add_(1, top, -scale * rows.gather(1, top))
        return param
    s = rows * rows + eps
    s = s / s.amax(dim=1, keepdim=True)
    q = s.pow(p_norm / 2 - 1)
    row_factor = (s * q).sum(dim=1, keepdim=True).pow(2 / p_norm - 1)
    rows.addcmul_(row_factor * q, rows, value=-scale)
    return param


def _adam_(param, grad, exp_avg, exp_avg_sq, lr, beta1, beta2, eps, step):
    exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    denom = (exp_avg_sq.sqrt() / math.sqrt(1 - beta2 ** step)).add_(eps)
    param.addcdiv_(exp_avg, denom, value=-lr / (1 - beta1 ** step))


def _fused_ok(*tensors):
    return all(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() for t in tensors)


class AdamW(Optimizer):
    """``AdamW(model, lr, betas, eps, weight_decay)``: takes the model, not a parameter list, because
    the decay of a parameter depends on the p of its module (one parameter group per parameter)."""

    def __init__(self, model, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2):
        for name, value, ok in (("learning rate", lr, lr >= 0.0), ("epsilon value", eps, eps >= 0.0),
                                ("beta parameter at index 0", betas[0], 0.0 <= betas[0] < 1.0),
                                ("beta parameter at index 1", betas[1], 0.0 <= betas[1] < 1.0),
                                ("weight_decay value", weight_decay, weight_decay >= 0.0)):
            if not ok:
                raise ValueError(f"Invalid {name}: {value}")
        groups = [{"params": [prm], "module": mod} for mod in model.modules()
                  for prm in mod.parameters(recurse=False)]
        super().__init__(groups, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            p_norm = get_p_norm(group["module"])
            beta1, beta2 = group["betas"]
            lr, eps, wd = group["lr"], group["eps"], group["weight_decay"]
            for prm in group["params"]:
                grad = prm.grad
                if grad is None:
                    continue
                if grad.is_sparse:
                    raise RuntimeError("AdamW does not support sparse gradients")
                state = self.state[prm]
                if not state:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros_like(prm, memory_format=torch.preserve_format)
                    state["exp_avg_sq"] = torch.zeros_like(prm, memory_format=torch.preserve_format)
                state["step"] += 1
                m, v = state["exp_avg"], state["exp_avg_sq"]
                if _fused_ok(prm, grad, m, v):
                    norm_dist_cpp.adamw_lp_step(prm, grad, m, v, p_norm, lr, beta1, beta2, eps, wd, state["step"])
                else:
                    lp_weight_decay_(prm, p_norm, lr, wd, eps)
                    _adam_(prm, grad, m, v, lr, beta1, beta2, eps, state["step"])
        return loss
