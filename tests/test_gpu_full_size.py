"""GPU parity at the full sizes of the benchmark configurations (BASELINE.json configs 0-4).

The vectorised oracle is fast enough to check the L_inf paths bit for bit at full
size; the p-norm and bound paths are checked on a row subset of the full-size
layer (rows are independent) plus size-independent invariants on the whole output.
"""
import math

import pytest
import torch

import oracle
from helpers import SIGN, assert_scatter_close, assert_sum_close, gen

pytestmark = pytest.mark.gpu


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
    # thousands of O(1) gradients can land on one input here; the kernels sum them in double and round once
    assert_scatter_close(gx.cpu(), oracle.inf_dist_backward_input(go, ep, ci, 1))
    assert_scatter_close(gw.cpu(), oracle.inf_dist_backward_weight(go, ep, ci, 1))
    # both gradients in one call: at this size one launch whose workgroups do either scatter
    gx2 = torch.full((512, ci, 1), float("nan"), device=DEV)
    gw2 = torch.full((5120, ci), float("nan"), device=DEV)
    cpp.inf_dist_backward_overwrite(go.to(DEV), pos.to(DEV), gx2, gw2, 1)
    torch.cuda.synchronize()
    assert torch.equal(gx2, gx) and torch.equal(gw2, gw)   # double bins: the rounded sums do not depend on the order


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


@pytest.mark.parametrize("ci", [3072, 5120])
def test_config2_backward_at_the_full_batch(ci):
    """Both p-norm gradients on the GPU at batch 512, from the one call the benchmark's step makes (at p = 8 the
    kernel that evaluates every term once for both sums) and from the two separate calls (the register-tiled
    kernels), compared with the oracle on 16 rows of grad_input (rows are independent) and 32 rows of grad_weight
    over all 512 images (each weight row is an independent reduction).  Reference: model/norm_dist_cuda.cu:299-425."""
    from gpu_common import DEV, cpp, gpu_norm_forward, say
    say("config 2 layer backward at batch 512:", ci, "-> 5120, p = 8")
    p = 8.0
    x, w = _layer(512, ci, 5120, seed=40 + ci)
    x = ((x - 0.47) / 0.2009).contiguous()
    out = gpu_norm_forward(x, w, 1, p)
    go = torch.randn(512, 5120, 1, generator=gen(41))
    gx = torch.empty(512, ci, 1, device=DEV)
    gw = torch.zeros(5120, ci, device=DEV)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV))
    cpp.norm_dist_backward_input(*args, gx, 1, p)
    cpp.norm_dist_backward_weight(*args, gw, 1, p)
    gx1 = torch.full((512, ci, 1), float("nan"), device=DEV)
    gw1 = torch.zeros(5120, ci, device=DEV)
    cpp.norm_dist_backward(*args, gx1, gw1, 1, p)
    torch.cuda.synchronize()
    gx, gw, gx1, gw1 = gx.cpu(), gw.cpu(), gx1.cpu(), gw1.cpu()
    expect_x = [(rows, oracle.norm_dist_backward_input(go[rows].contiguous(), x[rows].contiguous(), w, out[rows].contiguous(),
                                                       1, p, with_abs_terms=True))
                for rows in (slice(100, 116), slice(496, 512))]
    expect_w = [(slice(n0, n0 + 32), oracle.norm_dist_backward_weight(go[:, n0:n0 + 32].contiguous(), x, w[n0:n0 + 32].contiguous(),
                                                                      out[:, n0:n0 + 32].contiguous(), 1, p, with_abs_terms=True))
                for n0 in (0, 2077, 5088)]
    for name, tx, tw in (("separate calls", gx, gw), ("one call", gx1, gw1)):
        for rows, (ex, mx) in expect_x:
            say(" ", name, "grad_input rows", rows.start, "worst err/bound", round(assert_sum_close(tx[rows], ex, mx, p), 3))
        for cols, (ew, mw) in expect_w:
            say(" ", name, "grad_weight rows", cols.start, "worst err/bound", round(assert_sum_close(tw[cols], ew, mw, p), 3))
    # whole-tensor invariant (Euler: the norm is homogeneous of degree one in (x, w)):
    # sum x*grad_x + sum w*grad_w = sum g*out
    lhs = float((x.double().squeeze(-1) * gx.double().squeeze(-1)).sum() + (w.double() * gw.double()).sum())
    rhs = float((go.double() * out.double()).sum())
    scale = float((go.double() * out.double()).abs().sum())
    assert abs(lhs - rhs) <= 1e-5 * scale, (lhs, rhs, scale)


def _bench_mlp(p, train, batch):
    """The benchmark's own net, weights and inputs (bench.py: configs 1-3)."""
    import bench
    from gpu_common import DEV, pkg
    g = torch.Generator().manual_seed(0)
    img = torch.rand(batch, 3, 32, 32, generator=g)
    ws = bench.stack_weights(g)
    model = bench.build_mlp(pkg, ws, DEV, p, train=train)
    return bench, model, img, ws, g


def test_config1_whole_stack_training_step():
    """The whole 5-layer net of config 1 (training-mode mean shift, head as the benchmark builds it), one forward +
    backward on the GPU; every layer repeated by the oracle on what the GPU fed it (values bit-exact, both scatter
    gradients within rel 1e-5 / abs 1e-6, the arg-max indices bit for bit), and the oracle's own free-running stack against the last output.
    Reference: model/mlp.py:17-23, model/norm_dist.py:85-96."""
    from gpu_common import DEV, gpu_inf_forward, say
    from oracle import stack_check
    say("config 1: whole stack, batch 512, p = inf")
    bench, model, img, ws, g = _bench_mlp(float("inf"), True, 512)
    upstream = torch.randn(512, 10, generator=g)
    rep = stack_check.check_training_step(model, bench.normalise(img), upstream, float("inf"), DEV,
                                          inf_forward=lambda xs, ws: gpu_inf_forward(xs, ws, 1))
    say("  ", rep.as_json())
    assert rep.ok, rep.failures
    assert rep.exact == 15 and rep.toleranced >= 15     # per layer: values, the repeated launch, indices


def test_config2_whole_stack_training_step():
    """Config 2 (p = 8) through the whole net: every layer's forward on 16 batch rows, grad_input on the same rows and
    32 weight rows of grad_weight over the whole batch against the oracle, on the tensors the GPU really fed the layer."""
    from gpu_common import DEV, say
    from oracle import stack_check
    say("config 2: whole stack, batch 512, p = 8")
    bench, model, img, ws, g = _bench_mlp(8.0, True, 512)
    upstream = torch.randn(512, 10, generator=g)
    rep = stack_check.check_training_step(model, bench.normalise(img), upstream, 8.0, DEV, rows=slice(100, 116),
                                          weight_rows=slice(64, 96))
    say("  ", rep.as_json())
    assert rep.ok, rep.failures


def test_config3_whole_certification_pass_with_margins():
    """Config 3 end to end: values, lower and upper bounds through the five layers in evaluation mode (running means
    subtracted) and the certified margins of BoundFinalIdentity, bit for bit against the oracle's own pass
    (rows are independent in evaluation mode: 96 of the 1024 rows).  Reference: model/bound_module.py:95-103."""
    from gpu_common import DEV, pkg, say
    from oracle import stack_check
    say("config 3: whole certification pass, batch 1024 (96 rows compared)")
    bench, model, img, ws, g = _bench_mlp(float("inf"), False, 1024)
    means = [torch.randn(o, generator=g) * 0.1 for o in bench.LAYERS[1:]]
    with torch.no_grad():
        for layer, m in zip(list(model.fc) + [model.fc_last], means):
            layer.normalize.running_mean.copy_(m)
        model.fc_last.bias.copy_(torch.randn(10, generator=g) * 0.05)
    targets = torch.randint(0, 10, (1024,), generator=g)
    x, lo, up = (bench.normalise(t) for t in (img, (img - bench.EPS).clamp(0, 1), (img + bench.EPS).clamp(0, 1)))
    with torch.no_grad():
        y, l, u = model(x.to(DEV), lo.to(DEV), up.to(DEV))
        _, res = pkg.BoundFinalIdentity()(y, l, u, targets.to(DEV))
    torch.cuda.synchronize()
    rows = slice(400, 496)
    biases = [None] * 4 + [model.fc_last.bias.detach().cpu()]
    ey, el, eu, er = stack_check.oracle_certification(ws, means, biases, x[rows], lo[rows], up[rows], targets[rows])
    assert torch.equal(y.cpu()[rows], ey) and torch.equal(l.cpu()[rows], el) and torch.equal(u.cpu()[rows], eu)
    assert torch.equal(res.cpu()[rows], er)
    # on the whole batch: the value lies inside its bounds and the target's margin is zero
    assert bool((l <= y).all()) and bool((y <= u).all())
    assert bool((res.cpu().gather(1, targets.view(-1, 1)) == 0).all())


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
    # 131072 contributions per weight row, some 450 per element: summed in double, rounded once
    assert_scatter_close(gx.cpu(), oracle.inf_dist_backward_input(go, ep, 1152, 4))
    assert_scatter_close(gw.cpu(), oracle.inf_dist_backward_weight(go, ep, 1152, 4))


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
    expect = F.fold(oracle.inf_dist_backward_input_f64(go, ep, 1152, 4), (32, 32), 3, padding=1)
    assert_scatter_close(gimg.cpu(), expect)


def test_config4_layer_at_p8_from_the_image():
    """Config 4's layer in the p-norm phase, straight from the image at the full batch of 128.  The forward is
    checked on every image against this library's column kernel (bit for bit: the same arithmetic) and on the first
    four against the oracle; the gradients are taken for a grad_output that is zero outside the first four images, so
    that grad_weight of the full-size launch equals the oracle's on those four (rows are independent) and grad_img
    must be exactly zero everywhere else."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, say
    say("config 4 at p = 8 from the image: 128 x 128 x 32 x 32, 128 outputs, 4 groups")
    p, rows = 8.0, 4
    g = gen(9)
    img = torch.rand(128, 128, 32, 32, generator=g)
    w = (torch.randn(128, 288, generator=g) / math.sqrt(288)).contiguous()
    assert cpp.norm_dist_conv_supported(128, 32, 32, 128, 4, 3, 1, 1, 1)
    imgd, wd = img.to(DEV), w.to(DEV)
    out = torch.empty(128, 128, 1024, device=DEV)
    cpp.norm_dist_conv_forward(imgd, wd, out, 4, p, 3, 1, 1, 1)
    cols_d = torch.empty(128, 1152, 1024, device=DEV)
    cpp.unfold(imgd, cols_d, 3, 1, 1, 1)
    from_cols = torch.empty_like(out)
    cpp.norm_dist_forward(cols_d, wd, from_cols, 4, p)
    torch.cuda.synchronize()
    assert torch.equal(out, from_cols)
    del cols_d, from_cols
    cols = F.unfold(img[:rows], 3, padding=1).contiguous()
    ev = oracle.norm_dist_forward(cols, w, 4, p)
    torch.testing.assert_close(out[:rows].cpu(), ev, rtol=1e-5, atol=1e-6)

    go = torch.zeros(128, 128, 1024)
    go[:rows] = torch.randn(rows, 128, 1024, generator=g)
    gimg = torch.full((128, 128, 32, 32), float("nan"), device=DEV)
    gw = torch.zeros(128, 288, device=DEV)
    cpp.norm_dist_conv_backward_input(go.to(DEV), imgd, wd, out, gimg, 4, p, 3, 1, 1, 1)
    cpp.norm_dist_conv_backward_weight(go.to(DEV), imgd, wd, out, gw, 4, p, 3, 1, 1, 1)
    torch.cuda.synchronize()
    ex, mx = oracle.norm_dist_backward_input(go[:rows].contiguous(), cols, w, ev, 4, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go[:rows].contiguous(), cols, w, ev, 4, p, with_abs_terms=True)
    fold = lambda t: F.fold(t.double(), (32, 32), 3, padding=1)
    assert_sum_close(gimg[:rows].cpu(), fold(ex), fold(mx), p)
    assert bool((gimg[rows:] == 0).all())
    assert_sum_close(gw.cpu(), ew, mw, p)
