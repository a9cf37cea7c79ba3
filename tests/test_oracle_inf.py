"""Pins the oracle's L_inf forward and scatter backward (no GPU, no HIP library).

The reference holds no vectors for this path, so the pins are: hand-made
known answers for the tie / sign / zero rules, torch broadcasting closed forms
(sub, abs and max are exact in fp32, so equality is bit-for-bit), torch.cdist,
a pure-Python triple loop, and sum invariants of the scatter.
"""
import math

import pytest
import torch

import oracle
from helpers import (SIGN, closed_inf_forward, dense_inf_backward, gen, make_inputs, unpack_pos)


def fwd(x, w, G=1, literal=False):
    return oracle.inf_dist_forward(x, w, G, literal=literal)


# ---- known answers written by hand from the rule "strict >, k ascending" ---- #
KAT = [
    # x row, w row, expected out, expected pos
    ([0.0, 2.0], [1.0, 1.0], 1.0, 0 | SIGN),      # tie, first is x<w  -> lowest k, sign bit set
    ([2.0, 0.0], [1.0, 1.0], 1.0, 0),             # tie, first is x>w
    ([1.0, 1.0], [1.0, 1.0], 0.0, 0),             # all equal: nothing exceeds the initial 0
    ([0.0, 0.0, 5.0], [0.0, 0.0, 1.0], 4.0, 2),
    ([0.0, 0.0, 1.0], [0.0, 0.0, 5.0], 4.0, 2 | SIGN),
    ([3.0], [1.0], 2.0, 0),
    ([1.0], [3.0], 2.0, 0 | SIGN),
    ([-0.0, 0.0], [0.0, -0.0], 0.0, 0),           # signed zeros never win
    ([1.0, 4.0, 4.0, -2.0], [2.0, 1.0, 7.0, 1.0], 3.0, 1),  # three-way tie 3,3,3 -> k=1, positive
]


@pytest.mark.parametrize("literal", [True, False])
@pytest.mark.parametrize("xr,wr,eo,ep", KAT)
def test_known_answers(xr, wr, eo, ep, literal):
    x = torch.tensor(xr).reshape(1, -1, 1)
    w = torch.tensor(wr).reshape(1, -1)
    out, pos = fwd(x, w, literal=literal)
    assert out.item() == eo
    assert pos.item() == ep


@pytest.mark.parametrize("literal", [True, False])
def test_nan_never_wins_and_inf_does(literal):
    nan, inf = float("nan"), float("inf")
    x = torch.tensor([[nan, 1.0, 0.5], [nan, nan, nan], [0.0, inf, 2.0], [0.0, -inf, inf]]).reshape(4, 3, 1)
    w = torch.tensor([[0.0, 0.0, 0.0]])
    out, pos = fwd(x, w, literal=literal)
    assert out.flatten().tolist() == [1.0, 0.0, inf, inf]
    assert pos.flatten().tolist() == [1, 0, 1, 1 | SIGN]


SHAPES = [  # B, CO, CI, G, HW
    (3, 5, 1, 1, 1), (4, 7, 15, 1, 1), (4, 7, 17, 1, 1), (2, 3, 64, 1, 1), (2, 3, 65, 1, 1),
    (5, 6, 130, 1, 1), (3, 8, 24, 4, 1), (2, 6, 36, 3, 5), (2, 4, 18, 2, 7), (1, 1, 200, 1, 3),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("quant", [None, 4])
def test_matches_broadcast_closed_form(shape, quant):
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=sum(shape), quantize=quant)
    ev, ep = closed_inf_forward(x, w, G)
    for literal in (True, False):
        out, pos = fwd(x, w, G, literal=literal)
        assert torch.equal(out, ev)
        assert torch.equal(pos, ep)


def test_literal_equals_fast_under_heavy_ties():
    # coarse quantisation: most rows have many tied maxima spread over several 64-blocks
    x, w = make_inputs(16, 24, 777, 1, 1, seed=5, quantize=2)
    o1, p1 = fwd(x, w, literal=True)
    o2, p2 = fwd(x, w, literal=False)
    assert torch.equal(o1, o2) and torch.equal(p1, p2)
    idx, _ = unpack_pos(p1)
    assert int(idx.max()) < 777


def test_values_equal_cdist_config0_rows():
    # the MNIST-shaped config (K=784, 5120 outputs), on 32 of its 512 rows
    g = gen(0)
    x = torch.rand(512, 784, generator=g)[:32].contiguous()
    w = (torch.randn(5120, 784, generator=g) / math.sqrt(784)).contiguous()
    out, pos = fwd(x.reshape(32, 784, 1), w)
    ref = torch.cdist(x, w, p=float("inf"))
    assert torch.equal(out.reshape(32, 5120), ref)
    idx, neg = unpack_pos(pos.reshape(32, 5120))
    picked = x.gather(1, idx) - w.gather(1, idx.t()).t()
    assert torch.equal(picked.abs(), ref)
    assert torch.equal(picked < 0, neg)


def test_python_triple_loop_tiny():
    x, w = make_inputs(2, 4, 6, 2, 2, seed=11, quantize=8)
    out, pos = fwd(x, w, 2)
    K, NG = 3, w.shape[0] // 2
    for b in range(2):
        for n in range(w.shape[0]):
            g = n // NG
            for hw in range(2):
                best, bp = 0.0, 0
                for k in range(K):
                    t = x[b, g * K + k, hw].item() - w[n, k].item()
                    t = torch.tensor(t, dtype=torch.float32).item()
                    if abs(t) > best:
                        best, bp = abs(t), k | (SIGN if t < 0 else 0)
                assert out[b, n, hw].item() == pytest.approx(best, abs=0, rel=0)
                assert pos[b, n, hw].item() == bp


def test_bad_arguments_are_rejected():
    x = torch.zeros(2, 6, 1)
    w = torch.zeros(4, 2)  # 2*4 != 6 with G=4; CI % G != 0
    with pytest.raises(AssertionError):
        fwd(x, w, 4)
    lib = oracle.lib()
    assert lib.ldist_oracle_inf_dist_forward(None, None, 1, 1, 1, 1, 1, None, None) < 0
    assert lib.ldist_oracle_inf_dist_forward(None, None, 2, 4, 6, 4, 1, None, None) < 0


# ----------------------------- scatter backward ----------------------------- #
@pytest.mark.parametrize("shape", SHAPES)
def test_backward_matches_one_hot_expansion(shape):
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=1 + sum(shape), quantize=16)
    _, pos = fwd(x, w, G)
    go = torch.randn(B, CO, HW, generator=gen(3))
    ex, ew = dense_inf_backward(go, pos, CI, G)
    gx = oracle.inf_dist_backward_input(go, pos, CI, G)
    gw = oracle.inf_dist_backward_weight(go, pos, CI, G)
    torch.testing.assert_close(gx.double(), ex, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(gw.double(), ew, rtol=1e-6, atol=1e-7)
    # whole-tensor invariants: every (m,n) contributes +-g once to each gradient
    idx, neg = unpack_pos(pos)
    sg = torch.where(neg, -go, go).double()
    torch.testing.assert_close(gx.double().sum(), sg.sum(), rtol=1e-6, atol=1e-5)
    torch.testing.assert_close(gw.double().sum(), -sg.sum(), rtol=1e-6, atol=1e-5)
    assert int((gw != 0).sum(dim=1).max()) <= B * HW


def test_backward_collision_free_is_exact_and_signed():
    # every output points at its own input: sums have one term, so results are exact
    B, N, HW = 3, 5, 2
    K = N
    pos = torch.arange(N, dtype=torch.int32).reshape(1, N, 1).repeat(B, 1, HW).contiguous()
    pos[:, ::2, :] |= SIGN
    go = torch.randn(B, N, HW, generator=gen(9))
    gx = oracle.inf_dist_backward_input(go, pos, K, 1)
    sign = torch.where(pos < 0, -1.0, 1.0)
    assert torch.equal(gx, go * sign)
    # grad_w[n, n] = -sum_{b,hw} sign*g ; in double it is the same sum the oracle forms
    gw = oracle.inf_dist_backward_weight(go, pos, K, 1)
    expect = -(go.double() * sign.double()).sum(dim=(0, 2))
    torch.testing.assert_close(torch.diagonal(gw).double(), expect, rtol=1e-6, atol=1e-7)
    assert torch.count_nonzero(gw - torch.diag(torch.diagonal(gw))) == 0


def test_backward_accumulates_into_caller_buffer():
    x, w = make_inputs(4, 6, 10, 1, 1, seed=2)
    _, pos = fwd(x, w)
    go = torch.randn(4, 6, 1, generator=gen(4))
    base_x = torch.full((4, 10, 1), 0.5)
    base_w = torch.full((6, 10), -0.25)
    gx0 = oracle.inf_dist_backward_input(go, pos, 10, 1)
    gw0 = oracle.inf_dist_backward_weight(go, pos, 10, 1)
    gx1 = oracle.inf_dist_backward_input(go, pos, 10, 1, grad_input=base_x.clone())
    gw1 = oracle.inf_dist_backward_weight(go, pos, 10, 1, grad_weight=base_w.clone())
    torch.testing.assert_close(gx1, gx0 + 0.5)
    torch.testing.assert_close(gw1, gw0 - 0.25)


def test_forward_backward_finite_difference_tie_free():
    # d/dx and d/dw of sum(g * out) by central differences in float64 on a tie-free case
    B, N, K = 2, 3, 5
    g = gen(21)
    x = torch.rand(B, K, generator=g)
    w = torch.rand(N, K, generator=g)
    go = torch.randn(B, N, generator=g)
    _, pos = fwd(x.reshape(B, K, 1).contiguous(), w)
    gx = oracle.inf_dist_backward_input(go.reshape(B, N, 1).contiguous(), pos, K, 1).reshape(B, K)
    gw = oracle.inf_dist_backward_weight(go.reshape(B, N, 1).contiguous(), pos, K, 1)

    def f(xd, wd):
        return ((xd[:, None, :] - wd[None]).abs().amax(-1) * go.double()).sum()

    xd, wd = x.double(), w.double()
    h = 1e-6
    for b in range(B):
        for k in range(K):
            e = torch.zeros_like(xd); e[b, k] = h
            fd = (f(xd + e, wd) - f(xd - e, wd)) / (2 * h)
            assert abs(fd.item() - gx[b, k].item()) < 1e-5
    for n in range(N):
        for k in range(K):
            e = torch.zeros_like(wd); e[n, k] = h
            fd = (f(xd, wd + e) - f(xd, wd - e)) / (2 * h)
            assert abs(fd.item() - gw[n, k].item()) < 1e-5


@pytest.mark.parametrize("shape", [(3, 12, 10, 1, 1), (2, 8, 12, 2, 5), (4, 6, 9, 3, 7)])
def test_backward_input_f64_is_the_one_hot_expansion(shape):
    """oracle.inf_dist_backward_input_f64 (the column gradient left in float64, used where a check goes on summing
    before anything is rounded) against the dense one-hot expansion, exactly; its float32 rounding is the C oracle's."""
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=31, quantize=4)
    _, pos = oracle.inf_dist_forward(x, w, G)
    go = torch.randn(B, CO, HW, generator=gen(32))
    gx64 = oracle.inf_dist_backward_input_f64(go, pos, CI, G)
    dense_x, _ = dense_inf_backward(go, pos, CI, G)
    assert gx64.dtype == torch.float64 and torch.equal(gx64, dense_x)
    assert torch.equal(gx64.float(), oracle.inf_dist_backward_input(go, pos, CI, G))
