"""GPU parity at the full sizes of the benchmark configurations (BASELINE.json configs 0-4).

The vectorised oracle is fast enough to check the L_inf paths bit for bit at full
size; the p-norm and bound paths are checked on a row subset of the full-size
layer (rows are independent) plus size-independent invariants on the whole output.
"""
import math

import pytest
import torch

import oracle
from helpers import SIGN, assert_sum_close, gen

pytestmark = pytest.mark.gpu


def _scatter_magnitudes(go, pos, ci, G):
    """Sum of |g| landing on every gradient element: the scale of float32 rounding in the scatter sums."""
    mag_pos = pos & 0x7FFFFFFF                       # sign bit cleared: every contribution counts as +|g|
    mx = oracle.inf_dist_backward_input(go.abs(), mag_pos, ci, G)
    mw = -oracle.inf_dist_backward_weight(go.abs(), mag_pos, ci, G)
    return mx, mw


def _layer(B, CI, CO, seed=0):
    g = gen(seed)
    x = torch.rand(B, CI, 1, generator=g)
    w = (torch.randn(CO, CI, generator=g) / math.sqrt(CI)).contiguous()
    return x, w


def test_config0_forward_bit_exact():
    from gpu_common import gpu_inf_forward, say
    say("config 0: 512 x 784 -> 5120")
    x, w = _layer(512, 784, 5120)
    out, pos = gpu_inf_forward(x, w, 1)
    eo, ep = oracle.inf_dist_forward(x, w, 1)
    assert torch.equal(out, eo) and torch.equal(pos, ep)


@pytest.mark.parametrize("ci", [3072, 5120])
def test_config1_hidden_layer_forward_and_backward(ci):
    from gpu_common import DEV, cpp, gpu_inf_forward, say
    say("config 1 layer: 512 x", ci, "-> 5120")
    x, w = _layer(512, ci, 5120, seed=1)
    x = ((x - 0.47) / 0.2009).contiguous()           # normalised-image range, like the first layer's input
    out, pos = gpu_inf_forward(x, w, 1)
    eo, ep = oracle.inf_dist_forward(x, w, 1)
    assert torch.equal(out, eo) and torch.equal(pos, ep)
    go = torch.randn(512, 5120, 1, generator=gen(2))
    gx = torch.empty(512, ci, 1, device=DEV)
    gw = torch.empty(5120, ci, device=DEV)
    cpp.inf_dist_backward_input_overwrite(go.to(DEV), pos.to(DEV), gx, 1)
    cpp.inf_dist_backward_weight_overwrite(go.to(DEV), pos.to(DEV), gw, 1)
    torch.cuda.synchronize()
    # thousands of O(1) gradients can land on one input here: rel 1e-5 / abs 1e-6 relative to sum|g|
    mx, mw = _scatter_magnitudes(go, ep, ci, 1)
    assert_sum_close(gx.cpu(), oracle.inf_dist_backward_input(go, ep, ci, 1), mx)
    assert_sum_close(gw.cpu(), oracle.inf_dist_backward_weight(go, ep, ci, 1), mw)


def test_config1_head_forward_bit_exact():
    from gpu_common import gpu_inf_forward
    x, w = _layer(512, 5120, 10, seed=3)
    out, pos = gpu_inf_forward(x, w, 1)
    eo, ep = oracle.inf_dist_forward(x, w, 1)
    assert torch.equal(out, eo) and torch.equal(pos, ep)


def test_config2_pnorm_layer_rows_and_invariants():
    from gpu_common import DEV, cpp, gpu_norm_forward, say
    say("config 2 layer: 512 x 5120 -> 5120, p = 8")
    x, w = _layer(512, 5120, 5120, seed=4)
    p = 8.0
    out = gpu_norm_forward(x, w, 1, p)
    rows = slice(100, 116)
    torch.testing.assert_close(out[rows], oracle.norm_dist_forward(x[rows].contiguous(), w, 1, p), rtol=1e-5, atol=1e-6)
    # invariant on the whole output: a1 <= out <= K^(1/p) * a1 with a1 the L_inf distance
    a1, _ = oracle.inf_dist_forward(x, w, 1)
    assert bool((out >= a1 * (1 - 1e-6)).all()) and bool((out <= a1 * 5120 ** (1 / p) * (1 + 1e-6)).all())
    # gradients on the row subset (grad_input rows are independent; grad_weight of a row subset is a valid problem)
    go = torch.randn(16, 5120, 1, generator=gen(5))
    xs, outs = x[rows].contiguous(), out[rows].contiguous()
    ex, mx = oracle.norm_dist_backward_input(go, xs, w, outs, 1, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, xs, w, outs, 1, p, with_abs_terms=True)
    gx = torch.empty(16, 5120, 1, device=DEV)
    gw = torch.zeros(5120, 5120, device=DEV)
    args = (go.to(DEV), xs.to(DEV), w.to(DEV), outs.to(DEV))
    cpp.norm_dist_backward_input(*args, gx, 1, p)
    cpp.norm_dist_backward_weight(*args, gw, 1, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p)
    assert_sum_close(gw.cpu(), ew, mw, p)


def test_config3_bound_layer():
    from gpu_common import gpu_bound_forward, gpu_inf_forward, say
    say("config 3 layer: 1024 x 5120 -> 5120 bounds")
    x, w = _layer(1024, 5120, 5120, seed=6)
    eps = 8 / 255 / 0.2009
    lo, up = (x - eps).contiguous(), (x + eps).contiguous()
    ol, ou = gpu_bound_forward(lo, up, w, 1)
    rows = slice(500, 532)
    el, eu = oracle.inf_dist_bound_forward(lo[rows].contiguous(), up[rows].contiguous(), w, 1)
    assert torch.equal(ol[rows], el) and torch.equal(ou[rows], eu)
    # soundness on the whole output: L <= value(x) <= U, and U - L <= 2 eps (1-Lipschitz in L_inf)
    val, _ = gpu_inf_forward(x, w, 1)
    assert bool((ol <= val).all()) and bool((val <= ou).all())
    assert bool(((ou - ol) <= 2 * eps * (1 + 1e-5)).all())
    # the degenerate box reproduces the value forward bit for bit at full size
    dl, du = gpu_bound_forward(x, x, w, 1)
    assert torch.equal(dl, val) and torch.equal(du, val)


def test_config4_unfolded_conv_layer():
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, gpu_inf_forward, say
    say("config 4: 128 x 1152 x 1024, 128 outputs, 4 groups")
    g = gen(7)
    img = torch.rand(128, 128, 32, 32, generator=g)
    w = (torch.randn(128, 288, generator=g) / math.sqrt(288)).contiguous()
    cols = F.unfold(img, 3, padding=1).contiguous()
    out, pos = gpu_inf_forward(cols, w, 4)
    eo, ep = oracle.inf_dist_forward(cols, w, 4)
    assert torch.equal(out, eo) and torch.equal(pos, ep)
    go = torch.randn(128, 128, 1024, generator=g)
    gx = torch.empty(128, 1152, 1024, device=DEV)
    gw = torch.empty(128, 288, device=DEV)
    cpp.inf_dist_backward_input_overwrite(go.to(DEV), pos.to(DEV), gx, 4)
    cpp.inf_dist_backward_weight_overwrite(go.to(DEV), pos.to(DEV), gw, 4)
    torch.cuda.synchronize()
    # 131072 contributions per weight row: rel 1e-5 / abs 1e-6 relative to sum|g| per element
    mx, mw = _scatter_magnitudes(go, ep, 1152, 4)
    assert_sum_close(gx.cpu(), oracle.inf_dist_backward_input(go, ep, 1152, 4), mx)
    assert_sum_close(gw.cpu(), oracle.inf_dist_backward_weight(go, ep, 1152, 4), mw)


def test_config4_layer_from_the_image():
    """Config 4 without the unfolded tensor: forward and interval bounds straight from the images, and the input
    gradient written as an image, against the oracle on torch's columns (values, indices and bounds bit-exact)."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, say
    say("config 4 from the image: 128 x 128 x 32 x 32, 128 outputs, 4 groups")
    g = gen(8)
    img = torch.rand(128, 128, 32, 32, generator=g)
    w = (torch.randn(128, 288, generator=g) / math.sqrt(288)).contiguous()
    cols = F.unfold(img, 3, padding=1).contiguous()
    eo, ep = oracle.inf_dist_forward(cols, w, 4)
    out = torch.empty(128, 128, 1024, device=DEV)
    pos = torch.empty(128, 128, 1024, device=DEV, dtype=torch.int32)
    assert cpp.inf_dist_conv_forward_supported(128, 32, 32, 128, 4, 3, 1, 1, 1)
    cpp.inf_dist_conv_forward(img.to(DEV), w.to(DEV), out, pos, 4, 3, 1, 1, 1)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), eo) and torch.equal(pos.cpu(), ep)

    eps = 8.0 / 255
    lo_i, up_i = (img - eps).clamp(0, 1), (img + eps).clamp(0, 1)
    el, eu = oracle.inf_dist_bound_forward(F.unfold(lo_i, 3, padding=1).contiguous(),
                                           F.unfold(up_i, 3, padding=1).contiguous(), w, 4)
    ol, ou = torch.empty_like(out), torch.empty_like(out)
    cpp.inf_dist_bound_conv_forward(lo_i.to(DEV), up_i.to(DEV), w.to(DEV), ol, ou, 4, 3, 1, 1, 1)
    torch.cuda.synchronize()
    assert torch.equal(ol.cpu(), el) and torch.equal(ou.cpu(), eu)
    assert bool((el <= eo).all()) and bool((eo <= eu).all())     # the value lies inside its own bounds

    go = torch.randn(128, 128, 1024, generator=g)
    gimg = torch.empty(128, 128, 32, 32, device=DEV)
    cpp.inf_dist_backward_input_folded(go.to(DEV), pos, gimg, 4, 3, 1, 1, 1)
    torch.cuda.synchronize()
    gcols = oracle.inf_dist_backward_input(go, ep, 1152, 4)
    expect = F.fold(gcols.double(), (32, 32), 3, padding=1)
    terms = F.fold(oracle.inf_dist_backward_input(go.abs(), ep & ~SIGN, 1152, 4).double(), (32, 32), 3, padding=1).abs()
    assert_sum_close(gimg.cpu(), expect, terms)
