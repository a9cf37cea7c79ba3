"""Host-side behaviour of the Python layer (no GPU): dispatch, autograd contract, module semantics.

The native calls are replaced by fakes that run the CPU oracle on CPU tensors, so
what is tested here is the wrapper logic written from the reference's
model/norm_dist.py, model/mlp.py and model/bound_module.py -- not the kernels.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import __graft_entry__ as entry
import oracle
from helpers import gen

pkg = entry.load_package()
import l_inf_dist_net_amd.norm_dist_cpp as cpp  # noqa: E402  (module registered by load_package())


@pytest.fixture()
def fake_native(monkeypatch):
    calls = []

    def inf_dist_forward(x, w, out, pos, G):
        calls.append("inf_dist_forward")
        o, p = oracle.inf_dist_forward(x.contiguous(), w.contiguous(), G)
        out.copy_(o); pos.copy_(p)

    def inf_dist_forward_values(x, w, out, G):   # the fc layout only, like the library
        if x.size(2) != 1:
            return False
        calls.append("inf_dist_forward_values")
        out.copy_(oracle.inf_dist_forward(x.contiguous(), w.contiguous(), G)[0])
        return True

    def inf_dist_bound_forward(lo, up, w, ol, ou, G):
        calls.append("inf_dist_bound_forward")
        a, b = oracle.inf_dist_bound_forward(lo.contiguous(), up.contiguous(), w.contiguous(), G)
        ol.copy_(a); ou.copy_(b)

    def bwd_in_over(go, pos, gi, G):
        calls.append("inf_dist_backward_input_overwrite")
        gi.copy_(oracle.inf_dist_backward_input(go, pos, gi.size(1), G))

    def bwd_w_over(go, pos, gw, G):
        calls.append("inf_dist_backward_weight_overwrite")
        gw.copy_(oracle.inf_dist_backward_weight(go, pos, gw.size(1) * G, G))

    def bwd_both_over(go, pos, gi, gw, G):
        calls.append("inf_dist_backward_overwrite (input and weight)")
        gi.copy_(oracle.inf_dist_backward_input(go, pos, gi.size(1), G))
        gw.copy_(oracle.inf_dist_backward_weight(go, pos, gw.size(1) * G, G))

    def norm_dist_forward(x, w, out, G, p):
        calls.append("norm_dist_forward")
        out.copy_(oracle.norm_dist_forward(x.contiguous(), w.contiguous(), G, p))

    def norm_bwd_in(go, x, w, out, gi, G, p):
        calls.append("norm_dist_backward_input")
        gi.copy_(oracle.norm_dist_backward_input(go, x.contiguous(), w.contiguous(), out.contiguous(), G, p))

    def norm_bwd_w(go, x, w, out, gw, G, p):
        calls.append("norm_dist_backward_weight")
        assert torch.count_nonzero(gw) == 0  # the wrapper must hand over a zero-filled buffer
        oracle.norm_dist_backward_weight(go, x.contiguous(), w.contiguous(), out.contiguous(), G, p, grad_weight=gw)

    def norm_bwd_both(go, x, w, out, gi, gw, G, p):   # the one call that serves both gradients
        calls.append("norm_dist_backward (input and weight)")
        assert torch.count_nonzero(gw) == 0  # the wrapper must hand over a zero-filled buffer
        gi.copy_(oracle.norm_dist_backward_input(go, x.contiguous(), w.contiguous(), out.contiguous(), G, p))
        oracle.norm_dist_backward_weight(go, x.contiguous(), w.contiguous(), out.contiguous(), G, p, grad_weight=gw)

    monkeypatch.setattr(cpp, "norm_dist_backward", norm_bwd_both)
    for name, fn in [("inf_dist_forward", inf_dist_forward), ("inf_dist_forward_values", inf_dist_forward_values),
                     ("inf_dist_bound_forward", inf_dist_bound_forward),
                     ("inf_dist_backward_input_overwrite", bwd_in_over),
                     ("inf_dist_backward_weight_overwrite", bwd_w_over), ("inf_dist_backward_overwrite", bwd_both_over),
                     ("norm_dist_forward", norm_dist_forward),
                     ("norm_dist_backward_input", norm_bwd_in), ("norm_dist_backward_weight", norm_bwd_w)]:
        monkeypatch.setattr(cpp, name, fn)
    return calls


def test_binding_rejects_cpu_and_wrong_dtype_tensors():
    x, w = torch.zeros(2, 4, 1), torch.zeros(3, 4)
    out, pos = torch.zeros(2, 3, 1), torch.zeros(2, 3, 1, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):   # reference CHECK_CUDA, norm_dist.cpp:3
        cpp.inf_dist_forward(x, w, out, pos, 1)
    with pytest.raises(RuntimeError):
        cpp.norm_dist_forward(x, w, out, 1, 8.0)


def test_distf_dispatch_and_errors(fake_native):
    x = torch.rand(3, 6, 2, generator=gen(0))
    w = torch.rand(4, 3, generator=gen(1))
    y = pkg.norm_dist(x, w, 2, float("inf"))
    assert fake_native == ["inf_dist_forward"] and y.shape == (3, 4, 2)   # no gradient wanted, but not a layout the values-only call takes
    fake_native.clear()
    # fc layout: without a gradient to follow the forward skips the argmax; with one it records it
    xf, wf = torch.rand(3, 6, 1, generator=gen(2)), torch.rand(4, 3, generator=gen(3))
    y0 = pkg.norm_dist(xf, wf, 2, float("inf"))
    assert fake_native == ["inf_dist_forward_values"]
    fake_native.clear()
    y1 = pkg.norm_dist(xf.clone().requires_grad_(), wf, 2, float("inf"))
    assert fake_native == ["inf_dist_forward"] and torch.equal(y0, y1.detach())
    fake_native.clear()
    with torch.no_grad():
        pkg.norm_dist(xf.clone().requires_grad_(), wf, 2, float("inf"))
    assert fake_native == ["inf_dist_forward_values"]
    fake_native.clear()
    pkg.norm_dist(x, w, 2, 8.0)
    assert fake_native == ["norm_dist_forward"]
    with pytest.raises(NotImplementedError):       # model/norm_dist.py:21-22
        pkg.norm_dist(x, w, 2, 1.0)
    with pytest.raises(AssertionError):            # model/norm_dist.py:12
        pkg.norm_dist(x, w, 3, 8.0)


@pytest.mark.parametrize("p", [float("inf"), 8.0])
def test_distf_backward_respects_needs_input_grad(fake_native, p):
    x = torch.rand(3, 6, 2, generator=gen(2))
    w = torch.rand(4, 3, generator=gen(3))
    go = torch.randn(3, 4, 2, generator=gen(4))
    for rx, rw in ((True, True), (True, False), (False, True)):
        fake_native.clear()
        xx, ww = x.clone().requires_grad_(rx), w.clone().requires_grad_(rw)
        y = pkg.norm_dist(xx, ww, 2, p)
        y.backward(go.transpose(0, 1).contiguous().transpose(0, 1))  # a non-contiguous upstream gradient
        kinds = [c for c in fake_native if "backward" in c]
        assert any("input" in c for c in kinds) == rx and any("weight" in c for c in kinds) == rw
        assert (xx.grad is not None) == rx and (ww.grad is not None) == rw
        if rx and rw and not math.isinf(p):
            # both wanted: one call, for either layout and every exponent (the library decides inside it whether
            # one kernel serves both sums)
            assert kinds == ["norm_dist_backward (input and weight)"]
            for q in (p, 5.5, 2.0):
                fake_native.clear()
                x1, w1 = x[:, :, :1].clone().requires_grad_(True), w.clone().requires_grad_(True)
                pkg.norm_dist(x1, w1, 2, q).backward(go[:, :, :1].contiguous())
                assert [c for c in fake_native if "backward" in c] == ["norm_dist_backward (input and weight)"]
                assert x1.grad is not None and w1.grad is not None


def test_gradients_agree_with_the_dense_torch_formula(fake_native):
    # the reference's own cross-check: use_custom_cuda_func=False (model/norm_dist.py:52-57)
    x = torch.rand(4, 6, 3, generator=gen(5))
    w = torch.rand(4, 3, generator=gen(6))
    go = torch.randn(4, 4, 3, generator=gen(7))
    for p in (float("inf"), 6.0):
        a = [t.clone().requires_grad_(True) for t in (x, w)]
        b = [t.clone().requires_grad_(True) for t in (x, w)]
        ya = pkg.norm_dist(a[0], a[1], 2, p)
        yb = pkg.norm_dist(b[0], b[1], 2, p, use_custom_cuda_func=False)
        torch.testing.assert_close(ya, yb, rtol=1e-5, atol=1e-6)
        ya.backward(go); yb.backward(go)
        torch.testing.assert_close(a[0].grad, b[0].grad, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(a[1].grad, b[1].grad, rtol=1e-4, atol=1e-5)


def test_inf_dist_bound_matches_its_dense_formula(fake_native):
    x = torch.rand(4, 6, 3, generator=gen(8))
    w = torch.rand(4, 3, generator=gen(9))
    lo, up = (x - 0.1).contiguous(), (x + 0.1).contiguous()
    a = pkg.inf_dist_bound(lo, up, w, 2)
    b = pkg.inf_dist_bound(lo, up, w, 2, use_custom_cuda_func=False)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert not a[0].requires_grad


def test_mean_norm_train_and_eval():
    mn = pkg.MeanNorm(3, momentum=0.1)
    x = torch.randn(5, 3, 4, 4, generator=gen(10))
    mn.train()
    y = mn(x)
    mean = x.mean(dim=(0, 2, 3))
    torch.testing.assert_close(y, x - mean.view(1, 3, 1, 1))
    torch.testing.assert_close(mn.running_mean, 0.1 * mean)          # (1-m)*0 + m*mean, norm_dist.py:92-93
    mn.eval()
    torch.testing.assert_close(mn(x), x - mn.running_mean.view(1, 3, 1, 1))
    x2 = torch.randn(6, 3, generator=gen(11))                        # 2-D input path (norm_dist.py:90-91)
    mn.train()
    torch.testing.assert_close(mn(x2), x2 - x2.mean(dim=0))
    xg = x.clone().requires_grad_(True)                              # the batch mean carries gradient
    pkg.MeanNorm(3).train()(xg).sum().backward()
    torch.testing.assert_close(xg.grad, torch.zeros_like(x), atol=1e-6, rtol=0)
    # the hand-written backward of the shift against autograd through the plain formula, float64
    for shape in ((5, 3, 4, 4), (6, 3)):
        xa = torch.randn(*shape, generator=gen(12), dtype=torch.float64).requires_grad_(True)
        xb = xa.detach().clone().requires_grad_(True)
        up = torch.randn(*shape, generator=gen(13), dtype=torch.float64)
        pkg.MeanNorm(3).double().train()(xa).backward(up)
        dims = (0, 2, 3) if len(shape) == 4 else (0,)
        (xb - xb.mean(dim=dims, keepdim=True)).backward(up)
        torch.testing.assert_close(xa.grad, xb.grad, rtol=1e-12, atol=1e-12)


def naive_dist_conv(x, weight, stride, padding, group, p):
    """Direct loops over output positions: the definition the unfold-based layer must reproduce."""
    B, C, H, W = x.shape
    CO, CG, k, _ = weight.shape
    xp = F.pad(x, (padding,) * 4)
    oh, ow = (H + 2 * padding - k) // stride + 1, (W + 2 * padding - k) // stride + 1
    out = torch.zeros(B, CO, oh, ow)
    ng = CO // group
    for co in range(CO):
        g = co // ng
        for i in range(oh):
            for j in range(ow):
                patch = xp[:, g * CG:(g + 1) * CG, i * stride:i * stride + k, j * stride:j * stride + k]
                d = (patch - weight[co]).abs().reshape(B, -1)
                out[:, co, i, j] = d.max(dim=1)[0] if math.isinf(p) else (d.double() ** p).sum(1) ** (1 / p)
    return out


@pytest.mark.parametrize("p", [float("inf"), 4.0])
def test_conv_layer_matches_naive_loops(fake_native, p):
    torch.manual_seed(0)
    layer = pkg.NormDistConv(4, 6, 3, stride=2, padding=1, group=2, p=p, bias=True, mean_normalize=False)
    with torch.no_grad():
        layer.bias.copy_(torch.arange(6.0))
    x = torch.rand(2, 4, 5, 5, generator=gen(12))
    y, lo, up = layer(x)
    assert lo is None and up is None
    ref = naive_dist_conv(x, layer.weight.detach(), 2, 1, 2, p) + torch.arange(6.0).view(1, 6, 1, 1)
    torch.testing.assert_close(y, ref.float(), rtol=1e-5, atol=1e-6)


def test_fc_layer_is_a_1x1_conv_and_bounds_need_eval_and_inf(fake_native):
    torch.manual_seed(1)
    fc = pkg.NormDist(6, 5, p=float("inf"), bias=True, mean_normalize=True)
    x = torch.rand(4, 6, generator=gen(13))
    fc.eval()
    fc.normalize.running_mean.copy_(torch.linspace(-1, 1, 5))
    y, lo, up = fc(x, x - 0.05, x + 0.05)
    ev, _ = oracle.inf_dist_forward(x.reshape(4, 6, 1), fc.weight.detach().reshape(5, 6), 1)
    torch.testing.assert_close(y, ev.reshape(4, 5) - fc.normalize.running_mean + fc.bias)
    assert bool((lo <= y + 1e-6).all()) and bool((y <= up + 1e-6).all())
    el, eu = oracle.inf_dist_bound_forward((x - 0.05).reshape(4, 6, 1), (x + 0.05).reshape(4, 6, 1),
                                           fc.weight.detach().reshape(5, 6), 1)
    torch.testing.assert_close(lo, el.reshape(4, 5) - fc.normalize.running_mean + fc.bias)   # same shift on the bounds
    torch.testing.assert_close(up, eu.reshape(4, 5) - fc.normalize.running_mean + fc.bias)
    fc.train()
    with pytest.raises(AssertionError):            # model/norm_dist.py:143
        fc(x, x - 0.05, x + 0.05)
    fc.eval(); fc.p = 8.0
    with pytest.raises(AssertionError):
        fc(x, x - 0.05, x + 0.05)


def test_constructor_state_dict_and_p_setters():
    torch.manual_seed(2)
    conv = pkg.NormDistConv(4, 8, 3, group=2, bias=True, mean_normalize=True)
    assert sorted(conv.state_dict()) == ["bias", "normalize.running_mean", "weight"]
    assert conv.weight.shape == (8, 2, 3, 3) and conv.p == 0
    for i in range(8):                              # identity init, model/norm_dist.py:118-120
        assert conv.weight[i, i % 2, 1, 1].item() == -10.0
    wide = pkg.NormDistConv(8, 4, 1)                # in > out: no identity init
    assert not bool((wide.weight == -10.0).any())
    model = torch.nn.Sequential(pkg.NormDist(4, 4), torch.nn.ReLU(), pkg.NormDistConv(4, 4, 1))
    assert pkg.get_p_norm(model) == 0
    pkg.set_p_norm(model, 8.0)
    assert all(m.p == 8.0 for m in model if hasattr(m, "p")) and pkg.get_p_norm(model) == 8.0
    assert pkg.get_p_norm(torch.nn.Linear(2, 2)) is None
    t0 = pkg.NormDistConv.tag
    assert pkg.NormDist(2, 2).tag == t0 + 1
    # keyword spellings used by the benchmark description
    alias = pkg.NormDistConv(4, 8, 1, groups=2, mean_shift=True)
    assert alias.group == 2 and alias.normalize is not None
    assert pkg.MeanNormDist(4, 8).normalize is not None and pkg.MeanNormDist(4, 8).bias is None
    assert "in_features=4" in repr(pkg.NormDist(4, 8))


def test_mlp_triple_and_certified_margin(fake_native):
    torch.manual_seed(3)
    net = pkg.MLP(depth=3, width=1, input_dim=(3, 2, 2), num_classes=4)
    assert net.fc[0].out_channels == 1024            # width * 1024 hidden units, model/mlp.py:5
    pkg.set_p_norm(net, float("inf"))
    net.eval()
    x = torch.rand(5, 3, 2, 2, generator=gen(14))
    y, lo, up = net(x, x - 0.01, x + 0.01)
    assert y.shape == (5, 4) and bool((lo <= y + 1e-6).all()) and bool((y <= up + 1e-6).all())
    y_only = net(x)
    assert y_only[1] is None and y_only[2] is None and torch.equal(y_only[0], y)
    targets = torch.tensor([0, 1, 2, 3, 0])
    out, res = pkg.BoundFinalIdentity()(y, lo, up, targets)
    for b in range(5):
        for j in range(4):
            expect = 0.0 if j == targets[b] else (up[b, j] - lo[b, targets[b]]).item()
            assert res[b, j].item() == pytest.approx(expect)
    assert pkg.BoundFinalIdentity()(y) is y


def _tiny_model():
    torch.manual_seed(3)
    model = pkg.MLP(depth=2, width=1, input_dim=12, num_classes=5)
    model.extra = torch.nn.Linear(4, 3)            # a module without p: plain decay (reference adamw.py:42-43)
    return model


@pytest.mark.parametrize("p", [8.0, 2.0, 3.5, float("inf")])
def test_adamw_cpu_path_matches_oracle_per_parameter(p):
    """The optimizer's torch expressions (CPU tensors) against the C oracle, parameter by parameter,
    over three steps: group layout, step counter, state tensors, decay chosen by the owner's p."""
    import oracle
    model = _tiny_model()
    pkg.set_p_norm(model, p)
    opt = pkg.AdamW(model, lr=0.02, betas=(0.8, 0.95), eps=1e-7, weight_decay=0.4)
    owners = {id(g["params"][0]): g["module"] for g in opt.param_groups}
    assert len(opt.param_groups) == len(list(model.parameters()))           # one group per parameter
    mirror = {id(q): (q.detach().clone(), torch.zeros_like(q), torch.zeros_like(q)) for q in model.parameters()}
    g = gen(31)
    for step in (1, 2, 3):
        for q in model.parameters():
            q.grad = torch.randn(q.shape, generator=g)
        skipped = model.extra.bias
        skipped.grad = None                                                   # no gradient: untouched, no state
        before = skipped.detach().clone()
        opt.step()
        assert torch.equal(skipped.detach(), before) and len(opt.state[skipped]) == 0
        for q in model.parameters():
            if q.grad is None:
                continue
            w, m, v = mirror[id(q)]
            w2 = w.view(w.size(0), -1).contiguous()
            oracle.adamw_lp_step(w2, q.grad.reshape(w2.shape).contiguous(), m.view_as(w2), v.view_as(w2),
                                 pkg.get_p_norm(owners[id(q)]), 0.02, (0.8, 0.95), 1e-7, 0.4, step)
            w.copy_(w2.view_as(w))
            torch.testing.assert_close(q.detach(), w, rtol=2e-5, atol=1e-6)
            assert opt.state[q]["step"] == step
    assert pkg.get_p_norm(model.extra) is None


def test_adamw_constructor_checks_and_closure():
    model = _tiny_model()
    for bad in (dict(lr=-1.0), dict(eps=-1e-8), dict(betas=(1.0, 0.9)), dict(betas=(0.9, -0.1)), dict(weight_decay=-0.1)):
        with pytest.raises(ValueError):
            pkg.AdamW(model, **bad)
    pkg.set_p_norm(model, 8.0)
    opt = pkg.AdamW(model)
    calls = []

    def closure():
        calls.append(1)
        return torch.tensor(3.0)

    assert opt.step(closure).item() == 3.0 and calls == [1]


def test_model_wrapper_passes_bounds_only_with_targets():
    """Reference model/model.py:9-17: without targets the bounds are dropped; with targets and a feature that
    returns no bounds, the eps-ball around the feature output is what the predictor gets."""
    pkg = entry.load_package()
    seen = {}

    class Feature(torch.nn.Module):
        def forward(self, x, lower=None, upper=None):
            seen["feature"] = (lower, upper)
            return x * 2, None, None

    class Predictor(torch.nn.Module):
        def forward(self, x, lower, upper, targets=None):
            seen["predictor"] = (lower, upper, targets)
            return x

    net = pkg.Model(Feature(), Predictor(), eps=0.25)
    x = torch.ones(2, 3)
    net(x, lower=x - 1, upper=x + 1)
    assert seen["feature"] == (None, None) and seen["predictor"] == (None, None, None)
    t = torch.tensor([0, 1])
    net(x, lower=x - 1, upper=x + 1, targets=t)
    lo, up, tt = seen["predictor"]
    assert torch.equal(lo, x * 2 - 0.25) and torch.equal(up, x * 2 + 0.25) and tt is t
    pkg.set_eps(net, 0.5)
    assert pkg.get_eps(net) == 0.5 and pkg.get_eps(torch.nn.Linear(2, 2)) is None


def test_pgd_stays_in_the_ball_and_the_range_and_raises_the_loss():
    """Reference attack.py:15-36 on a plain linear classifier: the result lies within eps of the input and within
    [down, up], parameters get their requires_grad back, and the cross entropy does not go down."""
    pkg = entry.load_package()
    torch.manual_seed(3)
    net = torch.nn.Linear(12, 4)
    x = torch.rand(16, 12)
    y = torch.randint(0, 4, (16,))
    up, down = torch.ones(12), torch.zeros(12)
    adv = pkg.AttackPGD(net, eps=0.1, step_size=0.025, num_steps=8, up=up, down=down).find(x, y)
    assert float((adv - x).abs().max()) <= 0.1 + 1e-6
    assert float(adv.min()) >= 0.0 and float(adv.max()) <= 1.0
    assert all(p.requires_grad for p in net.parameters())
    ce = torch.nn.functional.cross_entropy
    with torch.no_grad():
        assert float(ce(net(adv), y)) >= float(ce(net(x), y))
    fixed = pkg.AttackPGD(net, 0.1, 0.025, 1, up, down, random_start=False).find(x, y)
    leaf = x.detach().clone().requires_grad_(True)
    ce(net(leaf), y, reduction="sum").backward()
    expect = torch.min(torch.max(leaf.detach() + 0.025 * leaf.grad.sign(), down), up)
    assert torch.allclose(fixed, expect)   # one step without the random start is the signed-gradient step


def test_certified_accuracy_clips_each_corner_on_one_side_only():
    """Reference main.py:178-179: lower = max(inputs - eps, down), upper = min(inputs + eps, up) -- the lower corner is
    not clipped from above nor the upper corner from below, which shows for inputs outside the data range."""
    pkg = entry.load_package()
    seen = {}

    class Net(torch.nn.Module):
        def forward(self, x, lower=None, upper=None, targets=None):
            seen["lower"], seen["upper"] = lower, upper
            return x, x

    x = torch.tensor([[-0.5, 0.2, 1.4], [0.05, 0.95, 0.5]])
    down, up = torch.zeros(3), torch.ones(3)
    pkg.certified_accuracy(Net(), x, torch.tensor([0, 1]), 0.1, up, down)
    assert torch.equal(seen["lower"], torch.max(x - 0.1, down)) and torch.equal(seen["upper"], torch.min(x + 0.1, up))
    assert float(seen["lower"][0, 2]) == pytest.approx(1.3) and float(seen["upper"][0, 0]) == pytest.approx(-0.4)


def test_train_step_and_accuracy_helpers():
    pkg = entry.load_package()
    torch.manual_seed(4)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = torch.nn.Linear(6, 3)

        def forward(self, x, targets=None):
            out = self.lin(x)
            return out, out - 0.1

    net = Net()
    opt = torch.optim.SGD(net.parameters(), lr=0.5)
    x, y = torch.randn(32, 6), torch.randint(0, 3, (32,))
    loss_fun = lambda out, worse, t: torch.nn.functional.cross_entropy(out, t)
    first, _ = pkg.train_step(net, loss_fun, opt, x, y)
    for _ in range(20):
        last, acc = pkg.train_step(net, loss_fun, opt, x, y)
    assert last < first and 0.0 <= acc <= 1.0
    assert pkg.cal_acc(torch.tensor([[0.1, 0.9], [0.8, 0.2]]), torch.tensor([1, 1])).tolist() == [1.0, 0.0]


@pytest.mark.parametrize("p", [float("inf"), 8.0])
def test_stack_checker_passes_on_a_correct_net_and_catches_a_wrong_one(fake_native, p):
    """The whole-stack checker (oracle/stack_check.py) on a small MLP on the CPU, native calls faked by the oracle:
    it must accept the correct net, and must notice a layer whose gradient routing or values were tampered with."""
    from oracle import stack_check
    torch.manual_seed(5)
    model = pkg.MLP(depth=3, width=1, input_dim=24, num_classes=10, head_mean_normalize=True)
    import l_inf_dist_net_amd.mlp as mlp_mod
    pkg.set_p_norm(model, p)
    model.train()
    x = torch.rand(12, 24, generator=gen(1))
    up = torch.randn(12, 10, generator=gen(2))
    rep = stack_check.check_training_step(model, x, up, p, torch.device("cpu"))
    assert rep.ok, rep.failures
    assert rep.toleranced >= 9 and (rep.exact == 3 if math.isinf(p) else rep.exact == 0)

    if math.isinf(p):
        # the direct comparison of the indices: the entry point run again on every recorded input
        def inf_forward(xs, ws, flip=False):
            o = torch.empty(xs.size(0), ws.size(0), 1)
            ps = torch.empty(xs.size(0), ws.size(0), 1, dtype=torch.int32)
            cpp.inf_dist_forward(xs, ws, o, ps, 1)
            if flip:
                ps[3, 2, 0] ^= 1          # one index off by one, value untouched
            return o, ps
        rep = stack_check.check_training_step(model, x, up, p, torch.device("cpu"), inf_forward=inf_forward)
        assert rep.ok and rep.exact == 9, rep.failures
        bad = stack_check.check_training_step(model, x, up, p, torch.device("cpu"),
                                              inf_forward=lambda a, b: inf_forward(a, b, flip=True))
        assert not bad.ok and all("arg-max indices" in f for f in bad.failures)

    # a wrong operator: values off by one ulp-sized factor in one layer
    good = cpp.inf_dist_forward if math.isinf(p) else cpp.norm_dist_forward

    def off_values(*a):
        good(*a)
        a[2].mul_(1.0 + 3e-5)
    name = "inf_dist_forward" if math.isinf(p) else "norm_dist_forward"
    setattr(cpp, name, off_values)
    try:
        bad = stack_check.check_training_step(model, x, up, p, torch.device("cpu"))
    finally:
        setattr(cpp, name, good)
    assert not bad.ok and any("values" in f for f in bad.failures)

    # a wrong gradient: grad_weight scaled
    wname = "inf_dist_backward_overwrite" if math.isinf(p) else "norm_dist_backward"   # both gradients are wanted: one call
    good_w = getattr(cpp, wname)

    def off_grad(*a):
        good_w(*a)
        (a[3] if math.isinf(p) else a[5]).mul_(1.001)   # the grad_weight argument of either call
    setattr(cpp, wname, off_grad)
    try:
        bad = stack_check.check_training_step(model, x, up, p, torch.device("cpu"))
    finally:
        setattr(cpp, wname, good_w)
    assert not bad.ok and any("grad_weight" in f for f in bad.failures)


def test_oracle_certification_matches_the_modules(fake_native):
    """oracle_certification (the free-running evaluation pass with margins) against the package's own MLP +
    BoundFinalIdentity driven by the faked native calls: same arithmetic, bit for bit."""
    from oracle import stack_check
    torch.manual_seed(6)
    model = pkg.MLP(depth=3, width=1, input_dim=24, num_classes=10, head_mean_normalize=True)
    pkg.set_p_norm(model, float("inf"))
    model.eval()
    layers = list(model.fc) + [model.fc_last]
    with torch.no_grad():
        for layer in layers:
            layer.normalize.running_mean.copy_(torch.randn(layer.out_channels) * 0.1)
        model.fc_last.bias.copy_(torch.randn(10) * 0.1)
    x = torch.rand(9, 24, generator=gen(3))
    lo, up = (x - 0.03).clamp(0, 1), (x + 0.03).clamp(0, 1)
    targets = torch.randint(0, 10, (9,), generator=gen(4))
    with torch.no_grad():
        y, l, u = model(x, lo, up)
        _, res = pkg.BoundFinalIdentity()(y, l, u, targets)
    ws = [ly.weight.detach().reshape(ly.weight.size(0), -1).contiguous() for ly in layers]
    means = [ly.normalize.running_mean.clone() for ly in layers]
    biases = [None, None, model.fc_last.bias.detach()]
    ey, el, eu, er = stack_check.oracle_certification(ws, means, biases, x, lo, up, targets)
    assert torch.equal(y, ey) and torch.equal(l, el) and torch.equal(u, eu) and torch.equal(res, er)
