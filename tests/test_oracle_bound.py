"""Pins the oracle's interval-bound forward (no GPU).

Pins: the broadcasting closed form, the equivalent spelling max(l-w, w-u, 0)
for l <= u, the degenerate box l = u = x (must reproduce the L_inf forward
bit-for-bit), soundness on sampled points of the box, and tightness by brute
force over the 2^K corners for tiny K.
"""
import itertools

import pytest
import torch

import oracle
from helpers import closed_bound, dense_diff, gen, make_inputs

SHAPES = [(3, 5, 1, 1, 1), (4, 7, 17, 1, 1), (2, 3, 65, 1, 1), (3, 8, 24, 4, 1), (2, 6, 36, 3, 5), (2, 4, 18, 2, 7)]


def box(x, eps):
    return (x - eps).clamp(0, 1).contiguous(), (x + eps).clamp(0, 1).contiguous()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("eps", [0.0, 8 / 255, 0.3])
def test_matches_closed_forms(shape, eps):
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=7 + sum(shape))
    lo_in, up_in = box(x, eps)
    lo, up = oracle.inf_dist_bound_forward(lo_in, up_in, w, G)
    el, eu = closed_bound(lo_in, up_in, w, G)
    assert torch.equal(lo, el) and torch.equal(up, eu)
    # second spelling, valid because lower <= upper: L = max_k max(l-w, w-u, 0)
    tl = dense_diff(lo_in, w, G)
    tu = dense_diff(up_in, w, G)
    alt = torch.maximum(torch.maximum(tl, -tu), torch.zeros_like(tl)).amax(dim=3).reshape(B, CO, HW)
    assert torch.equal(lo, alt)  # torch.equal treats +0 and -0 as equal
    alt_u = torch.maximum(tl.abs(), tu.abs()).amax(dim=3).reshape(B, CO, HW)
    assert torch.equal(up, alt_u)


@pytest.mark.parametrize("shape", SHAPES)
def test_degenerate_box_reproduces_forward(shape):
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=sum(shape))
    val, _ = oracle.inf_dist_forward(x, w, G)
    lo, up = oracle.inf_dist_bound_forward(x, x, w, G)
    assert torch.equal(lo, val) and torch.equal(up, val)


def test_soundness_and_monotonicity():
    B, CO, CI, G, HW = 6, 9, 40, 1, 1
    x, w = make_inputs(B, CO, CI, G, HW, seed=3)
    prev_l = prev_u = None
    for eps in (0.01, 0.05, 0.2):
        lo_in, up_in = box(x, eps)
        lo, up = oracle.inf_dist_bound_forward(lo_in, up_in, w, G)
        g = gen(17)
        for _ in range(20):
            xp = (lo_in + (up_in - lo_in) * torch.rand(x.shape, generator=g)).contiguous()
            v, _ = oracle.inf_dist_forward(xp, w, G)
            assert bool((lo <= v).all()) and bool((v <= up).all())
        if prev_l is not None:
            assert bool((lo <= prev_l).all()) and bool((up >= prev_u).all())
        prev_l, prev_u = lo, up


def test_tight_at_box_corners_tiny_k():
    # U is attained at a corner; L is the minimum over the box of a convex function per
    # coordinate, so it equals the minimum over points built from {l, u, clamp(w)} per k.
    K, N = 4, 3
    g = gen(5)
    x = torch.rand(1, K, 1, generator=g)
    w = torch.rand(N, K, generator=g)
    lo_in, up_in = box(x, 0.15)
    lo, up = oracle.inf_dist_bound_forward(lo_in, up_in, w, 1)
    l, u = lo_in.flatten(), up_in.flatten()
    for n in range(N):
        best_u = 0.0
        for corner in itertools.product([0, 1], repeat=K):
            pt = torch.where(torch.tensor(corner, dtype=torch.bool), u, l)
            best_u = max(best_u, (pt - w[n]).abs().max().item())
        assert up[0, n, 0].item() == best_u
        pt = torch.minimum(torch.maximum(w[n], l), u)  # closest point of the box to w[n]
        assert lo[0, n, 0].item() == pytest.approx((pt - w[n]).abs().max().item(), abs=1e-7)


def test_nan_is_ignored_like_fmax():
    nan = float("nan")
    l = torch.tensor([[nan, 0.2]]).reshape(1, 2, 1)
    u = torch.tensor([[nan, 0.4]]).reshape(1, 2, 1)
    w = torch.tensor([[0.0, 0.0]])
    lo, up = oracle.inf_dist_bound_forward(l, u, w, 1)
    assert lo.item() == pytest.approx(0.2) and up.item() == pytest.approx(0.4)
