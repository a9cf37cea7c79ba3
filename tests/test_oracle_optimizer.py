"""Pins for the two oracle functions outside the reference's native module: the per-channel mean
shift (MeanNorm, reference model/norm_dist.py:85-96) and the AdamW step with row-wise l_p weight
decay (reference adamw.py:36-85).  None of the checks retypes the oracle's formula: the decay is
checked against autograd of ||w||_p^2 / 2, special cases with closed answers (p = 2, p = inf,
one-element rows) and invariants; the Adam part against torch.optim.Adam."""
import math

import pytest
import torch

import oracle
from helpers import gen

HP = dict(lr=0.05, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.3)


def decay_only(w, p_norm, **kw):
    hp = {**HP, **kw}
    out = w.clone()
    oracle.adamw_lp_step(out, None, None, None, p_norm, hp["lr"], hp["betas"], hp["eps"], hp["weight_decay"], 1)
    return out


def test_mean_shift_against_float64_and_momentum():
    x = torch.randn(7, 5, 6, generator=gen(1)) + torch.arange(5.0).view(1, 5, 1)
    running = torch.linspace(-1, 1, 5)
    before = running.clone()
    y, mean = oracle.mean_shift(x, running, momentum=0.25)
    m64 = x.double().mean(dim=(0, 2))
    torch.testing.assert_close(mean.double(), m64, rtol=1e-7, atol=1e-7)
    torch.testing.assert_close(y.double(), x.double() - m64.view(1, 5, 1), rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(running.double(), 0.75 * before.double() + 0.25 * m64, rtol=1e-6, atol=1e-7)
    assert y.mean(dim=(0, 2)).abs().max() < 1e-6                   # the shifted tensor has zero channel means
    y2, _ = oracle.mean_shift(y)                                     # idempotent up to rounding
    torch.testing.assert_close(y2, y, rtol=0, atol=1e-6)


def test_decay_p2_is_plain_multiplicative_decay():
    w = torch.randn(9, 40, generator=gen(2))
    torch.testing.assert_close(decay_only(w, 2.0), w * (1 - HP["lr"] * HP["weight_decay"]), rtol=1e-6, atol=1e-8)
    torch.testing.assert_close(decay_only(w, None), w * (1 - HP["lr"] * HP["weight_decay"]), rtol=1e-6, atol=1e-8)


def test_decay_inf_touches_only_the_first_largest_entry_of_each_row():
    w = torch.randn(6, 30, generator=gen(3))
    w[2, 5], w[2, 17] = 4.0, -4.0                                    # a tie: the first one decays
    out = decay_only(w, float("inf"))
    expect = w.clone()
    top = w.abs().argmax(dim=1)
    assert top[2].item() == 5
    for r in range(6):
        expect[r, top[r]] = w[r, top[r]] * (1 - HP["lr"] * HP["weight_decay"])
    torch.testing.assert_close(out, expect, rtol=1e-6, atol=0)
    assert (out != w).sum().item() == 6


@pytest.mark.parametrize("p", [3.0, 4.0, 8.0, 5.5, 37.0])
def test_decay_is_the_gradient_of_half_the_squared_p_norm(p):
    # d/dw (||w||_p^2 / 2) = ||w||_p^(2-p) |w|^(p-2) w; the oracle's eps only regularises zeros
    w = (torch.randn(5, 24, generator=gen(4)) * 0.7 + 0.1)
    w64 = w.double().requires_grad_(True)
    (0.5 * w64.abs().pow(p).sum(dim=1).pow(2.0 / p)).sum().backward()
    expect = w.double() - HP["lr"] * HP["weight_decay"] * w64.grad
    torch.testing.assert_close(decay_only(w, p, eps=1e-30).double(), expect, rtol=2e-6, atol=1e-7)


def test_decay_invariants():
    w = torch.randn(4, 50, generator=gen(5))
    for p in (3.0, 8.0, 21.0):
        a = decay_only(w, p, eps=1e-30)
        # rows are independent
        torch.testing.assert_close(decay_only(w[1:2].contiguous(), p, eps=1e-30), a[1:2], rtol=0, atol=0)
        # scale equivariance: the decay of c*w is c times the decay of w
        torch.testing.assert_close(decay_only(3.0 * w, p, eps=1e-30), 3.0 * a, rtol=2e-6, atol=1e-7)
        # sign symmetry and shrinkage: no entry grows or changes sign
        torch.testing.assert_close(decay_only(-w, p, eps=1e-30), -a, rtol=0, atol=0)
        assert torch.all(a.abs() <= w.abs()) and torch.all(a * w >= 0)
        # Euler: sum_i w_i * (w_i - a_i) = lr*wd * ||w||_p^2
        lhs = (w.double() * (w.double() - a.double())).sum(dim=1)
        rhs = HP["lr"] * HP["weight_decay"] * w.double().abs().pow(p).sum(dim=1).pow(2.0 / p)
        torch.testing.assert_close(lhs, rhs, rtol=1e-5, atol=1e-8)
    # one-element rows (biases): every p gives plain decay
    b = torch.randn(12, 1, generator=gen(6))
    for p in (None, 3.0, 8.0, float("inf")):
        torch.testing.assert_close(decay_only(b, p), b * (1 - HP["lr"] * HP["weight_decay"]), rtol=1e-6, atol=1e-9)
    # large p approaches the p = inf rule on a row with a clear maximum
    r = torch.tensor([[0.1, -0.2, 3.0, 0.5]])
    torch.testing.assert_close(decay_only(r, 400.0), decay_only(r, float("inf")), rtol=1e-5, atol=1e-7)


def test_adam_part_matches_torch_optim_adam():
    w0 = torch.randn(6, 10, generator=gen(7))
    ref = w0.clone().requires_grad_(True)
    opt = torch.optim.Adam([ref], lr=HP["lr"], betas=HP["betas"], eps=HP["eps"])
    w, m, v = w0.clone(), torch.zeros_like(w0), torch.zeros_like(w0)
    for step in range(1, 6):
        g = torch.randn(6, 10, generator=gen(100 + step))
        ref.grad = g.clone()
        opt.step()
        oracle.adamw_lp_step(w, g, m, v, None, HP["lr"], HP["betas"], HP["eps"], 0.0, step)   # no decay
        torch.testing.assert_close(w, ref.detach(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(m, opt.state[ref]["exp_avg"], rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(v, opt.state[ref]["exp_avg_sq"], rtol=1e-6, atol=1e-9)


def test_decay_comes_before_adam_and_acts_on_the_parameter():
    # with a zero gradient Adam moves nothing, so a full step equals the decay alone
    w = torch.randn(3, 16, generator=gen(8))
    full, m, v = w.clone(), torch.zeros_like(w), torch.zeros_like(w)
    oracle.adamw_lp_step(full, torch.zeros_like(w), m, v, 8.0, HP["lr"], HP["betas"], HP["eps"], HP["weight_decay"], 1)
    torch.testing.assert_close(full, decay_only(w, 8.0), rtol=0, atol=0)
    assert torch.count_nonzero(m) == 0 and torch.count_nonzero(v) == 0
