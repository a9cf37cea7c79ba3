"""Pins the oracle's p-norm forward and backward (no GPU).

Pins: float64 closed form, torch.cdist (library routine, fc layout), p = 2
(Euclidean), bounds a1 <= out <= K^(1/p) a1, homogeneity, monotonicity in p,
convergence to L_inf, robustness to scale (the max-normalised stabilisation),
torch.autograd through the closed form for both gradients, and Euler's
identity for a degree-1 homogeneous function.
"""
import pytest
import torch

import oracle
from helpers import closed_pnorm, gen, make_inputs

SHAPES = [(3, 5, 1, 1, 1), (4, 7, 17, 1, 1), (2, 3, 65, 1, 1), (3, 8, 24, 4, 1), (2, 6, 36, 3, 5), (2, 4, 18, 2, 7)]
PS = [1.5, 2.0, 3.0, 8.0, 37.5, 1000.0]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", PS)
def test_forward_matches_float64_closed_form(shape, p):
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=13 + sum(shape))
    out = oracle.norm_dist_forward(x, w, G, p)
    torch.testing.assert_close(out.double(), closed_pnorm(x, w, G, p), rtol=2e-7, atol=1e-12)


@pytest.mark.parametrize("p", [2.0, 3.0, 8.0])
def test_forward_matches_cdist(p):
    g = gen(1)
    x = torch.rand(9, 300, generator=g)
    w = torch.randn(11, 300, generator=g) / 300 ** 0.5
    out = oracle.norm_dist_forward(x.reshape(9, 300, 1).contiguous(), w, 1, p).reshape(9, 11)
    ref = torch.cdist(x.double(), w.double(), p=p)
    torch.testing.assert_close(out.double(), ref, rtol=2e-7, atol=0)
    if p == 2.0:
        eu = ((x.double()[:, None] - w.double()[None]) ** 2).sum(-1).sqrt()
        torch.testing.assert_close(out.double(), eu, rtol=2e-7, atol=0)


def test_forward_invariants():
    B, CO, CI, G, HW = 4, 6, 50, 1, 1
    x, w = make_inputs(B, CO, CI, G, HW, seed=2)
    a1, _ = oracle.inf_dist_forward(x, w, G)
    prev = None
    for p in (2.0, 4.0, 8.0, 64.0, 512.0, 4096.0):
        out = oracle.norm_dist_forward(x, w, G, p)
        assert bool((out >= a1 * (1 - 1e-6)).all())
        assert bool((out <= a1 * (CI ** (1.0 / p)) * (1 + 1e-6)).all())
        if prev is not None:
            assert bool((out <= prev * (1 + 1e-6)).all())  # decreasing in p
        prev = out
        c = -3.5  # homogeneity of degree one
        outc = oracle.norm_dist_forward((x * c).contiguous(), (w * c).contiguous(), G, p)
        torch.testing.assert_close(outc, out * abs(c), rtol=1e-6, atol=0)
    torch.testing.assert_close(prev, a1, rtol=2e-3, atol=0)  # p = 4096 is within K^(1/p) of L_inf


@pytest.mark.parametrize("scale", [1e-20, 1e-6, 1.0, 1e6, 1e18])
def test_forward_is_scale_robust(scale):
    x, w = make_inputs(3, 4, 33, 1, 1, seed=4)
    base = closed_pnorm(x, w, 1, 8.0)
    out = oracle.norm_dist_forward((x * scale).contiguous(), (w * scale).contiguous(), 1, 8.0)
    if scale >= 1e-6:
        torch.testing.assert_close(out.double(), base * scale, rtol=1e-6, atol=0)
    else:
        # below the reference's 1e-10 seed the seed dominates: result is finite, positive, tiny
        assert bool(torch.isfinite(out).all()) and bool((out > 0).all()) and bool((out < 1e-9).all())


def test_all_equal_inputs_give_the_seed_value():
    # x == w everywhere: out = 1e-10 * (1e-10)^(1/p)  (reference seeds, norm_dist_cuda.cu:232-233,289)
    x = torch.full((1, 8, 1), 0.25)
    w = torch.full((2, 8), 0.25)
    out = oracle.norm_dist_forward(x, w, 1, 8.0)
    assert out.flatten().tolist() == pytest.approx([1e-10 * 1e-10 ** (1 / 8)] * 2, rel=1e-6)


def test_float_reference_order_variant_is_close():
    x, w = make_inputs(8, 16, 784, 1, 1, seed=6)
    for p in (8.0, 100.0):
        a = oracle.norm_dist_forward(x, w, 1, p)
        b = oracle.norm_dist_forward(x, w, 1, p, f32_reference_order=True)
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)


def autograd_grads(x, w, G, p, go):
    xd = x.double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    out = closed_pnorm(xd, wd, G, p)
    out.backward(go.double())
    return out.detach(), xd.grad, wd.grad


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [1.5, 2.0, 3.0, 8.0, 37.5])
def test_backward_matches_autograd(shape, p):
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=29 + sum(shape))
    go = torch.randn(B, CO, HW, generator=gen(8))
    out64, ex, ew = autograd_grads(x, w, G, p, go)
    out = oracle.norm_dist_forward(x, w, G, p)
    gx = oracle.norm_dist_backward_input(go, x, w, out, G, p)
    gw = oracle.norm_dist_backward_weight(go, x, w, out, G, p)
    # `out` enters the backward rounded to float: (|t|/out)^(p-1) moves by (p-1)*6e-8 relative
    tol = 4e-7 * max(p, 2.0)
    scale_x = (go.abs().double().sum(dim=1, keepdim=True) if CO else 1)
    torch.testing.assert_close(gx.double(), ex, rtol=tol, atol=tol * float(go.abs().sum()) / B)
    torch.testing.assert_close(gw.double(), ew, rtol=tol, atol=tol * float(go.abs().sum()) / CO)


def test_backward_weight_accumulates():
    x, w = make_inputs(3, 4, 10, 1, 1, seed=3)
    go = torch.randn(3, 4, 1, generator=gen(2))
    out = oracle.norm_dist_forward(x, w, 1, 4.0)
    g0 = oracle.norm_dist_backward_weight(go, x, w, out, 1, 4.0)
    g1 = oracle.norm_dist_backward_weight(go, x, w, out, 1, 4.0, grad_weight=torch.full_like(w, 2.0))
    torch.testing.assert_close(g1, g0 + 2.0)


@pytest.mark.parametrize("p", [3.0, 8.0])
def test_euler_identity_and_antisymmetry(p):
    # out is homogeneous of degree 1 in (x, w):  <x, grad_x> + <w, grad_w> = <g, out>
    B, CO, CI, G, HW = 5, 6, 24, 2, 3
    x, w = make_inputs(B, CO, CI, G, HW, seed=31)
    go = torch.randn(B, CO, HW, generator=gen(5))
    out = oracle.norm_dist_forward(x, w, G, p)
    gx = oracle.norm_dist_backward_input(go, x, w, out, G, p).double()
    gw = oracle.norm_dist_backward_weight(go, x, w, out, G, p).double()
    lhs = (x.double() * gx).sum() + (w.double() * gw).sum()
    rhs = (go.double() * out.double()).sum()
    torch.testing.assert_close(lhs, rhs, rtol=1e-5, atol=1e-6)
    # out depends on x - w only: the two gradients cancel in total
    torch.testing.assert_close(gx.sum(), -gw.sum(), rtol=1e-5, atol=1e-6)


def test_euler_identity_holds_for_the_linf_pair_too():
    B, CO, CI, G, HW = 5, 6, 24, 2, 3
    x, w = make_inputs(B, CO, CI, G, HW, seed=37)
    go = torch.randn(B, CO, HW, generator=gen(6))
    out, pos = oracle.inf_dist_forward(x, w, G)
    gx = oracle.inf_dist_backward_input(go, pos, CI, G).double()
    gw = oracle.inf_dist_backward_weight(go, pos, CI, G).double()
    lhs = (x.double() * gx).sum() + (w.double() * gw).sum()
    torch.testing.assert_close(lhs, (go.double() * out.double()).sum(), rtol=1e-5, atol=1e-6)


def test_rejects_p_not_above_one():
    x, w = make_inputs(1, 1, 2, 1, 1)
    with pytest.raises(RuntimeError):
        oracle.norm_dist_forward(x, w, 1, 1.0)
