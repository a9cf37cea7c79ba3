#!/usr/bin/env python3
"""Benchmark of the distance-neuron hot path on one MI355X.

Default workload (BASELINE.json configs[1], the one the metric is quoted on): the
CIFAR-10-shaped 5-layer L_inf-dist MLP 3072 -> 5120 -> 5120 -> 5120 -> 5120 -> 10 at
p = inf, batch 512, fp32, forward plus backward (grad_x of every layer and every
grad_w).  A "step" is one pass of the hot path over one synthetic batch that already
sits in HBM.  `--workload c0|c2|c3|c4` runs the other BASELINE.json configurations
(`c4i`: configs[4] from the image, `c4p`: the same layer at finite p from the image, `c1t`: configs[1] with the
optimizer step) with the
same output format (they are parity-test cases; the driver's line is c1).

Prints ONE JSON line.  `value` is G dist-ops/s; a dist-op is one (row, output,
input) triple of one pass (forward, grad-input or grad-weight for the p-norm paths;
the forward only at p = inf, whose backward is a byte-bound scatter).  `roofline`
is measured live on the workload's dominant kernel with events on the stream the
kernels run on; `cpu_baseline` times the CPU oracle on a bounded row sample of the
same workload.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

LAYERS = [3072, 5120, 5120, 5120, 5120, 10]
CIFAR_MEAN = (0.4914, 0.4822, 0.4465)
CIFAR_STD = 0.2009
EPS = 8 / 255
FP32_PEAK_TFLOPS = 157.3          # MI355X vector fp32 peak (counts packed FMA)
INF = float("inf")


def stack_ops(batch):
    return sum(batch * a * b for a, b in zip(LAYERS[:-1], LAYERS[1:]))


def normalise(x):
    import torch
    mean = torch.tensor(CIFAR_MEAN).view(1, 3, 1, 1)
    return ((x - mean) / CIFAR_STD).reshape(x.size(0), -1).contiguous()


def stack_weights(g):
    import torch
    return [torch.randn(o, i, generator=g) / math.sqrt(i) for i, o in zip(LAYERS[:-1], LAYERS[1:])]


def build_mlp(pkg, ws, dev, p, train):
    import torch
    model = pkg.MLP(depth=5, width=5, input_dim=3072, num_classes=10, head_mean_normalize=True)
    with torch.no_grad():
        for layer, w in zip(list(model.fc) + [model.fc_last], ws):
            layer.weight.copy_(w.view_as(layer.weight))
    pkg.set_p_norm(model, p)
    model = model.to(dev)
    return model.train() if train else model.eval()


class KernelTimer:
    """Brackets every launch of one binding function with events on the current stream."""

    def __init__(self, cpp, torch, name, flops_of, accept):
        self.cpp, self.torch, self.name, self.flops_of, self.accept = cpp, torch, name, flops_of, accept
        self.orig = getattr(cpp, name)
        self.records = []
        self.enabled = False

    def __enter__(self):
        def timed(*args):
            if not self.enabled or not self.accept(*args):
                return self.orig(*args)
            a = self.torch.cuda.Event(enable_timing=True)
            b = self.torch.cuda.Event(enable_timing=True)
            a.record()
            self.orig(*args)
            b.record()
            self.records.append((a, b, self.flops_of(*args)))
        setattr(self.cpp, self.name, timed)
        return self

    def __exit__(self, *exc):
        setattr(self.cpp, self.name, self.orig)

    def summary(self):
        ms = sum(a.elapsed_time(b) for a, b, _ in self.records)
        flops = sum(f for _, _, f in self.records)
        n = len(self.records)
        return n, ms / max(n, 1), flops / max(n, 1)


def mnk(x, w):
    return x.size(0) * x.size(2) * w.size(0) * w.size(1)


# --------------------------------------------------------------------------- #
# Workloads.  Each gives: step(), dist-ops per step, images per step, a CPU     #
# sample function, and the kernel to time for the roofline: (binding name,      #
# flops per launch, launch filter, description, algorithmic flops per dist-op). #
# --------------------------------------------------------------------------- #
def workload_c0(pkg, torch, dev):
    g = torch.Generator().manual_seed(0)
    x = torch.rand(512, 784, generator=g).reshape(512, 784, 1).contiguous()
    w = (torch.randn(5120, 784, generator=g) / math.sqrt(784)).contiguous()
    xd, wd = x.to(dev), w.to(dev)
    out = torch.empty(512, 5120, 1, device=dev)
    pos = torch.empty(512, 5120, 1, device=dev, dtype=torch.int32)
    cpp = pkg.norm_dist_cpp

    def step():
        cpp.inf_dist_forward(xd, wd, out, pos, 1)

    def cpu(oracle, rows):
        oracle.inf_dist_forward(x[:rows].contiguous(), w, 1)
        return rows * 784 * 5120

    def formula(rows):
        pkg.norm_dist(x[:rows].contiguous(), w, 1, INF, use_custom_cuda_func=False)
        return rows * 784 * 5120

    def check(oracle, stack_check):
        rep = stack_check.Report()
        step()
        torch.cuda.synchronize()
        ev, ep = oracle.inf_dist_forward(x, w, 1)
        rep.equal("values", out.cpu(), ev)
        rep.equal("argmax index and sign", pos.cpu(), ep)
        return rep

    return dict(step=step, ops=512 * 784 * 5120, images=512, full_rows=512, cpu=cpu, formula=formula, check=check,
                name="configs[0]: single L_inf-dist fc layer forward, 512 x 784 -> 5120, values + argmax",
                kernel=("inf_dist_forward", lambda x_, w_, *_: 2 * mnk(x_, w_), lambda *a: True,
                        "inf_forward_kernel (tiled L_inf forward)", 2))


def mlp_workload(pkg, torch, dev, p):
    g = torch.Generator().manual_seed(0)
    x = normalise(torch.rand(512, 3, 32, 32, generator=g))
    ws = stack_weights(g)
    upstream = torch.randn(512, 10, generator=g)
    model = build_mlp(pkg, ws, dev, p, train=True)
    xd = x.to(dev).requires_grad_(True)
    up = upstream.to(dev)

    def step():
        xd.grad = None
        for prm in model.parameters():
            prm.grad = None
        y, _, _ = model(xd)
        y.backward(up)

    def cpu(oracle, rows):
        h = x[:rows].reshape(rows, -1, 1).contiguous()
        saved = []
        for w in ws:
            if math.isinf(p):
                out, pos = oracle.inf_dist_forward(h, w, 1)
            else:
                out, pos = oracle.norm_dist_forward(h, w, 1, p), None
            saved.append((h, w, out, pos))
            h = (out - out.mean(dim=0, keepdim=True)).contiguous()
        gr = upstream[:rows].reshape(rows, -1, 1).contiguous()
        for (hin, w, out, pos) in reversed(saved):
            gr = (gr - gr.mean(dim=0, keepdim=True)).contiguous()
            if math.isinf(p):
                oracle.inf_dist_backward_weight(gr, pos, hin.size(1), 1)
                gr = oracle.inf_dist_backward_input(gr, pos, hin.size(1), 1)
            else:
                oracle.norm_dist_backward_weight(gr, hin, w, out, 1, p)
                gr = oracle.norm_dist_backward_input(gr, hin, w, out, 1, p)
        return stack_ops(rows) * (1 if math.isinf(p) else 3)

    def formula(rows):
        # forward + backward through the dense torch formula (what the reference runs with
        # use_custom_cuda_func=False), autograd doing the backward
        import torch
        h = x[:rows].reshape(rows, -1, 1).clone().requires_grad_(True)
        params = [w.clone().requires_grad_(True) for w in ws]
        out = h
        for w in params:
            out = pkg.norm_dist(out, w, 1, p, use_custom_cuda_func=False)
            out = out - out.mean(dim=0, keepdim=True)
        out.backward(upstream[:rows].reshape(rows, -1, 1))
        return stack_ops(rows) * (1 if math.isinf(p) else 3)

    def check(oracle, stack_check):
        # one training step of the whole stack, every layer repeated by the oracle on what the GPU really fed it:
        # p = inf on the full batch; p-norm (slow on the CPU) on 16 batch rows and 32 weight rows per layer
        if math.isinf(p):
            def inf_forward(xs, ws):      # the library's forward entry point on a recorded layer input
                o = torch.empty(xs.size(0), ws.size(0), 1, device=dev)
                ps = torch.empty(xs.size(0), ws.size(0), 1, device=dev, dtype=torch.int32)
                pkg.norm_dist_cpp.inf_dist_forward(xs.to(dev), ws.to(dev), o, ps, 1)
                torch.cuda.synchronize()
                return o.cpu(), ps.cpu()
            return stack_check.check_training_step(model, x, upstream, p, dev, inf_forward=inf_forward)
        return stack_check.check_training_step(model, x, upstream, p, dev, rows=slice(100, 116), weight_rows=slice(64, 96))

    return step, cpu, formula, check


def workload_c1(pkg, torch, dev):
    step, cpu, formula, check = mlp_workload(pkg, torch, dev, INF)
    return dict(step=step, ops=stack_ops(512), images=512, full_rows=512, cpu=cpu, formula=formula, check=check,
                name="configs[1]: 5-layer L_inf-dist MLP 3072-5120-5120-5120-5120-10, p=inf, batch 512, "
                     "forward+backward (all grad_x and grad_w), mean shift in training mode",
                kernel=("inf_dist_forward", lambda x_, w_, *_: 2 * mnk(x_, w_),
                        lambda x_, w_, o_, p_, G: w_.size(0) // G > 16,   # the 10-way head runs another kernel
                        "inf_forward_kernel (tiled L_inf forward)", 2))


def workload_c1t(pkg, torch, dev):
    # configs[1] followed by the optimizer: one complete training step of the reference's recipe
    # (main.py: forward, backward, AdamW with l_inf weight decay), on the same synthetic batch
    g = torch.Generator().manual_seed(0)
    x = normalise(torch.rand(512, 3, 32, 32, generator=g))
    ws = stack_weights(g)
    upstream = torch.randn(512, 10, generator=g)
    model = build_mlp(pkg, ws, dev, INF, train=True)
    opt = pkg.AdamW(model, lr=1e-3, weight_decay=5e-3)
    xd, up = x.to(dev), upstream.to(dev)

    def step():
        for prm in model.parameters():
            prm.grad = None
        y, _, _ = model(xd)
        y.backward(up)
        opt.step()

    base = workload_c1(pkg, torch, dev)
    return dict(base, step=step,
                name="configs[1] plus the AdamW step with l_inf weight decay: one full training step "
                     "(forward, backward, optimizer) of the 5-layer MLP, batch 512")


C2_P = 8.0   # --p moves it along the reference's annealing schedule (8 ... 1000); the configuration itself is p = 8


def workload_c2(pkg, torch, dev):
    step, cpu, formula, check = mlp_workload(pkg, torch, dev, C2_P)
    return dict(step=step, ops=3 * stack_ops(512), images=512, full_rows=512, cpu=cpu, formula=formula, check=check,
                name=f"configs[2]: the same MLP at p={C2_P:g}, forward+backward (3 dist-op passes per layer)",
                kernel=("norm_dist_backward_input", lambda go, x_, w_, *_: 7 * mnk(x_, w_),
                        lambda go, x_, w_, *_: w_.size(0) > 16,
                        "norm_backward_input_tiled_kernel (grad_input, register-tiled)", 7)
                if C2_P == 2.0 else   # the exponent whose two register-tiled kernels beat the one-pass kernel
                       ("norm_dist_backward", lambda go, x_, w_, *_: 2 * 7 * mnk(x_, w_),
                        lambda go, x_, w_, *_: w_.size(0) > 16,
                        "norm_backward_fused_kernel (both gradients from one evaluation of every term; the flops are "
                        "those of the two sums as the reference computes them)", 7))


def workload_c3(pkg, torch, dev):
    g = torch.Generator().manual_seed(0)
    img = torch.rand(1024, 3, 32, 32, generator=g)
    x, lo, up = normalise(img), normalise((img - EPS).clamp(0, 1)), normalise((img + EPS).clamp(0, 1))
    ws = stack_weights(g)
    means = [torch.randn(o, generator=g) * 0.1 for o in LAYERS[1:]]
    model = build_mlp(pkg, ws, dev, INF, train=False)
    with torch.no_grad():
        for layer, m in zip(list(model.fc) + [model.fc_last], means):
            layer.normalize.running_mean.copy_(m)
    targets = torch.randint(0, 10, (1024,), generator=g).to(dev)
    final = pkg.BoundFinalIdentity()
    xd, lod, upd = x.to(dev), lo.to(dev), up.to(dev)

    def step():
        with torch.no_grad():
            y, l, u = model(xd, lod, upd)
            return final(y, l, u, targets)

    def cpu(oracle, rows):
        h, l, u = (t[:rows].reshape(rows, -1, 1).contiguous() for t in (x, lo, up))
        for w, m in zip(ws, means):
            out, _ = oracle.inf_dist_forward(h, w, 1)
            ol, ou = oracle.inf_dist_bound_forward(l, u, w, 1)
            h, l, u = ((t - m.view(1, -1, 1)).contiguous() for t in (out, ol, ou))
        return 2 * stack_ops(rows)

    def formula(rows):
        h, l, u = (t[:rows].reshape(rows, -1, 1).contiguous() for t in (x, lo, up))
        for w, m in zip(ws, means):
            out = pkg.norm_dist(h, w, 1, INF, use_custom_cuda_func=False)
            ol, ou = pkg.inf_dist_bound(l, u, w, 1, use_custom_cuda_func=False)
            h, l, u = ((t - m.view(1, -1, 1)).contiguous() for t in (out, ol, ou))
        return 2 * stack_ops(rows)

    def check(oracle, stack_check, rows=64):
        # evaluation mode: rows are independent and the shift by the running mean is one exact subtraction, so the
        # oracle's free-running pass must reproduce values, both bounds and the certified margins bit for bit
        rep = stack_check.Report()
        with torch.no_grad():
            y, l, u = model(xd[:rows], lod[:rows], upd[:rows])
            _, res = final(y, l, u, targets[:rows])
        torch.cuda.synchronize()
        biases = [None] * 4 + [model.fc_last.bias.detach().cpu()]
        ey, el, eu, er = stack_check.oracle_certification(ws, means, biases, x[:rows], lo[:rows], up[:rows],
                                                          targets[:rows].cpu())
        rep.equal("values", y.cpu(), ey)
        rep.equal("lower bounds", l.cpu(), el)
        rep.equal("upper bounds", u.cpu(), eu)
        rep.equal("certified margins", res.cpu(), er)
        return rep

    return dict(step=step, ops=2 * stack_ops(1024), images=1024, full_rows=1024, cpu=cpu, formula=formula, check=check,
                name="configs[3]: interval-bound certification forward through the MLP, batch 1024, eps=8/255: "
                     "value path + lower/upper bounds + certified margins (bound-ops and dist-ops both counted)",
                kernel=("inf_dist_bound_forward", lambda l_, u_, w_, *_: 6 * mnk(l_, w_),
                        lambda l_, u_, w_, *_: w_.size(0) > 16,   # the 10-way head runs another kernel
                        "bound_forward_kernel (tiled interval-bound forward)", 6))


def workload_c4(pkg, torch, dev):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(0)
    img = torch.rand(128, 128, 32, 32, generator=g)
    w = (torch.randn(128, 32, 3, 3, generator=g) / math.sqrt(288)).reshape(128, 288).contiguous()
    go = torch.randn(128, 128, 1024, generator=g)
    cols = F.unfold(img, 3, padding=1).contiguous()        # (128, 1152, 1024), outside the timed region
    xd = cols.to(dev).requires_grad_(True)
    wd = w.to(dev).requires_grad_(True)
    god = go.to(dev)

    def step():
        xd.grad = None
        wd.grad = None
        y = pkg.norm_dist(xd, wd, 4, INF)
        y.backward(god)

    def cpu(oracle, rows):
        xs, gs = cols[:rows].contiguous(), go[:rows].contiguous()
        _, pos = oracle.inf_dist_forward(xs, w, 4)
        oracle.inf_dist_backward_input(gs, pos, 1152, 4)
        oracle.inf_dist_backward_weight(gs, pos, 1152, 4)
        return rows * 1024 * 128 * 288

    def formula(rows):
        xs = cols[:rows].clone().requires_grad_(True)
        wr = w.clone().requires_grad_(True)
        pkg.norm_dist(xs, wr, 4, INF, use_custom_cuda_func=False).backward(go[:rows])
        return rows * 1024 * 128 * 288

    imgd = img.to(dev)
    layer = pkg.NormDistConv(128, 128, 3, padding=1, group=4, p=INF, bias=False, mean_normalize=False).to(dev)
    with torch.no_grad():
        layer.weight.copy_(w.view_as(layer.weight))
    god4 = god.view(128, 128, 32, 32)

    def step_from_image():
        # the layer as a user calls it: image in, image gradient out (native unfold, scatter and fold fused)
        layer.weight.grad = None
        xi = imgd.detach().requires_grad_(True)
        y, _, _ = layer(xi)
        y.backward(god4)

    def step_torch_unfold():
        # the same through torch's unfold and autograd's fold, as the reference's layer does it
        wd.grad = None
        xi = imgd.detach().requires_grad_(True)
        y = pkg.norm_dist(F.unfold(xi, 3, padding=1), wd, 4, INF)
        y.backward(god)

    def check(oracle, stack_check, rows=4):
        # the first images of the batch (rows are independent; grad_weight of a batch subset is a valid problem),
        # through the column kernels and through the layer that works on the image
        rep = stack_check.Report()
        xs, gs = cols[:rows].contiguous(), go[:rows].contiguous()
        ev, ep = oracle.inf_dist_forward(xs, w, 4)
        egx = oracle.inf_dist_backward_input(gs, ep, 1152, 4)
        egw = oracle.inf_dist_backward_weight(gs, ep, 1152, 4)
        xs_d = xs.to(dev).requires_grad_(True)
        w_d = w.to(dev).requires_grad_(True)
        y = pkg.norm_dist(xs_d, w_d, 4, INF)
        y.backward(gs.to(dev))
        rep.equal("columns: values", y.detach().cpu(), ev)
        pos_d = torch.empty(rows, 128, 1024, device=dev, dtype=torch.int32)
        pkg.norm_dist_cpp.inf_dist_forward(xs_d.detach(), w_d.detach(), torch.empty(rows, 128, 1024, device=dev), pos_d, 4)
        rep.equal("columns: arg-max indices and signs", pos_d.cpu(), ep)
        rep.ratio("columns: grad_input", stack_check.close_ratio(xs_d.grad.cpu(), egx), xs_d.grad.cpu(), egx)
        rep.ratio("columns: grad_weight", stack_check.close_ratio(w_d.grad.cpu(), egw), w_d.grad.cpu(), egw)
        layer.weight.grad = None
        xi = imgd[:rows].detach().requires_grad_(True)
        yi, _, _ = layer(xi)
        yi.backward(god4[:rows])
        rep.equal("image: values", yi.detach().cpu().reshape(rows, 128, 1024), ev)
        egi = F.fold(oracle.inf_dist_backward_input_f64(gs, ep, 1152, 4), (32, 32), 3, padding=1)
        rep.ratio("image: grad_image", stack_check.close_ratio(xi.grad.cpu(), egi), xi.grad.cpu(), egi)
        rep.ratio("image: grad_weight", stack_check.close_ratio(layer.weight.grad.cpu().reshape(128, 288), egw),
                  layer.weight.grad.cpu().reshape(128, 288), egw)
        layer.weight.grad = None
        return rep

    return dict(step=step, ops=128 * 1024 * 128 * 288, images=128, full_rows=128, cpu=cpu, formula=formula, check=check,
                layer_routes=lambda: layer.last_route,     # what NormDistConv's last forward took (image / columns)
                step_alt=[("ms_per_step_from_image", step_from_image),
                          ("ms_per_step_with_torch_unfold_and_fold", step_torch_unfold)],
                name="configs[4]: unfolded 3x3 L_inf-dist conv layer, batch 128, 128->128 channels, 32x32, groups 4, "
                     "forward+backward (unfold outside the timed region)",
                kernel=("inf_dist_forward", lambda x_, w_, *_: 2 * mnk(x_, w_), lambda *a: True,
                        "inf_forward_shortk_kernel (conv layout, the whole reduction of a tile resident in LDS)", 2))


def workload_c4i(pkg, torch, dev):
    """configs[4] as a user of the layer runs it: the image goes in and the image gradient comes out; the
    unfolded tensor and its gradient are never built (forward straight from the image, scatter and fold fused)."""
    wl = workload_c4(pkg, torch, dev)
    from_image = dict(wl["step_alt"])["ms_per_step_from_image"]
    cpp = pkg.norm_dist_cpp
    geometry = (128, 32, 32, 128, 4, 3, 1, 1, 1)
    # which kernels the layer's forward takes (a geometry the image kernel does not cover falls back to unfold + columns)
    wl["routes"] = {"forward_from_image": bool(cpp.inf_dist_conv_forward_supported(*geometry)),
                    "backward_input_from_image": True}
    wl.update(step=from_image,
              step_alt=[("ms_per_step_columns_only_unfold_outside", wl["step"]),
                        ("ms_per_step_with_torch_unfold_and_fold", dict(wl["step_alt"])["ms_per_step_with_torch_unfold_and_fold"])],
              name="configs[4] from the image: 3x3 L_inf-dist conv layer, batch 128, 128->128 channels, 32x32, groups 4, "
                   "forward+backward with patch extraction and its adjoint inside the timed region",
              kernel=("inf_dist_conv_forward", lambda img_, w_, o_, *_: 2 * o_.numel() * w_.size(1), lambda *a: True,
                      "inf_conv_forward_kernel (L_inf forward straight from the image, a group's image rows resident "
                      "in LDS)", 2))
    return wl


C4_P = 8.0   # --p moves it, as for c2


def workload_c4p(pkg, torch, dev):
    """configs[4]'s layer in the p-norm phase of training (the reference's conv recipe spends most epochs at finite
    p): the image goes in and the image gradient comes out, straight from the image."""
    import torch.nn.functional as F
    p = C4_P
    g = torch.Generator().manual_seed(0)
    img = torch.rand(128, 128, 32, 32, generator=g)
    w = (torch.randn(128, 32, 3, 3, generator=g) / math.sqrt(288)).reshape(128, 288).contiguous()
    go = torch.randn(128, 128, 1024, generator=g)
    imgd, god4 = img.to(dev), go.to(dev).view(128, 128, 32, 32)
    layer = pkg.NormDistConv(128, 128, 3, padding=1, group=4, p=p, bias=False, mean_normalize=False).to(dev)
    with torch.no_grad():
        layer.weight.copy_(w.view_as(layer.weight))

    def step():
        layer.weight.grad = None
        xi = imgd.detach().requires_grad_(True)
        y, _, _ = layer(xi)
        y.backward(god4)

    def step_columns():
        # the same layer through the native unfold, the column kernels and the native fold
        layer.finite_p_route = "columns"
        try:
            step()
        finally:
            layer.finite_p_route = "image"

    wd = w.to(dev).requires_grad_(True)

    def step_torch_unfold():
        # through torch's unfold and autograd's fold, as the reference's layer does it
        wd.grad = None
        xi = imgd.detach().requires_grad_(True)
        y = pkg.norm_dist(F.unfold(xi, 3, padding=1), wd, 4, p)
        y.backward(god4.view(128, 128, 1024))

    def cpu(oracle, rows):
        xs, gs = F.unfold(img[:rows], 3, padding=1).contiguous(), go[:rows].contiguous()
        out = oracle.norm_dist_forward(xs, w, 4, p)
        oracle.norm_dist_backward_input(gs, xs, w, out, 4, p)
        oracle.norm_dist_backward_weight(gs, xs, w, out, 4, p)
        return 3 * rows * 1024 * 128 * 288

    def formula(rows):
        xs = F.unfold(img[:rows], 3, padding=1).requires_grad_(True)
        wr = w.clone().requires_grad_(True)
        pkg.norm_dist(xs, wr, 4, p, use_custom_cuda_func=False).backward(go[:rows])
        return 3 * rows * 1024 * 128 * 288

    def check(oracle, stack_check, rows=4):
        rep = stack_check.Report()
        xs, gs = F.unfold(img[:rows], 3, padding=1).contiguous(), go[:rows].contiguous()
        ev = oracle.norm_dist_forward(xs, w, 4, p)
        egx, mgx = oracle.norm_dist_backward_input(gs, xs, w, ev, 4, p, with_abs_terms=True)
        egw, mgw = oracle.norm_dist_backward_weight(gs, xs, w, ev, 4, p, with_abs_terms=True)
        layer.weight.grad = None
        xi = imgd[:rows].detach().requires_grad_(True)
        yi, _, _ = layer(xi)
        yi.backward(god4[:rows])
        torch.cuda.synchronize()
        got = yi.detach().cpu().reshape(rows, 128, 1024)
        rep.ratio("image: values", stack_check.close_ratio(got, ev), got, ev)
        egi = F.fold(egx.double(), (32, 32), 3, padding=1)
        mgi = F.fold(mgx.double(), (32, 32), 3, padding=1)
        rep.ratio("image: grad_image", stack_check.sum_ratio(xi.grad.cpu(), egi, mgi, p), xi.grad.cpu(), egi)
        gw = layer.weight.grad.cpu().reshape(128, 288)
        rep.ratio("image: grad_weight", stack_check.sum_ratio(gw, egw, mgw, p), gw, egw)
        layer.weight.grad = None
        return rep

    return dict(step=step, ops=3 * 128 * 1024 * 128 * 288, images=128, full_rows=128, cpu=cpu, formula=formula,
                check=check,
                # a geometry the image kernels do not cover would fall back to unfold + columns + fold
                routes={"from_image": bool(pkg.norm_dist_cpp.norm_dist_conv_supported(128, 32, 32, 128, 4, 3, 1, 1, 1)),
                        "finite_p_route": layer.finite_p_route},
                layer_routes=lambda: layer.last_route,
                step_alt=[("ms_per_step_native_unfold_columns_fold", step_columns),
                          ("ms_per_step_with_torch_unfold_and_fold", step_torch_unfold)],
                name=f"configs[4]'s layer at p={p:g} from the image: 3x3 p-norm dist conv layer, batch 128, 128->128 "
                     "channels, 32x32, groups 4, forward+backward (3 dist-op passes), no unfolded tensor",
                kernel=("norm_dist_conv_backward", lambda go_, img_, w_, o_, *_: 2 * 7 * o_.numel() * w_.size(1),
                        lambda *a: True,
                        "norm_conv_backward_kernel (both gradients from one evaluation of every term, straight from the "
                        "image; the flops are those of the two sums as the reference computes them)", 7))


WORKLOADS = {"c0": workload_c0, "c1": workload_c1, "c1t": workload_c1t, "c2": workload_c2, "c3": workload_c3,
             "c4": workload_c4, "c4i": workload_c4i, "c4p": workload_c4p}


def cpu_baseline(wl, target_seconds=12.0):
    """The CPU oracle (C, OpenMP) on a row subset of the same workload, sized to about target_seconds."""
    import oracle
    probe = max(1, min(8, wl["full_rows"]))
    t0 = time.perf_counter()
    wl["cpu"](oracle, probe)
    t = time.perf_counter() - t0
    rows = int(max(probe, min(wl["full_rows"], probe * target_seconds / max(t, 1e-3))))
    ops, t, reps = 0, 0.0, 0
    while reps == 0 or (t < target_seconds and reps < 64):   # fast hosts: repeat until the sample is long enough
        t0 = time.perf_counter()
        ops += wl["cpu"](oracle, rows)
        t += time.perf_counter() - t0
        reps += 1
    return {
        "value": round(ops / t / 1e9, 3),
        "unit": "G dist-ops/s",
        "cores": oracle.num_threads(),
        "kind": "port",
        "sample": f"C oracle (OpenMP) on {rows} of {wl['full_rows']} rows of the same workload, "
                  f"{reps} pass(es), {t:.1f} s",
    }


def cpu_formula_baseline(wl, target_seconds=5.0):
    """The dense torch formula of the reference's use_custom_cuda_func=False path on the host CPU,
    on a few rows of the same workload (it materialises rows x N x K floats per layer)."""
    import torch
    rows = 1 if wl["full_rows"] <= 128 else 2
    t0 = time.perf_counter()
    ops = wl["formula"](rows)
    t = time.perf_counter() - t0
    reps = 1
    while t < target_seconds and reps < 256:
        t0 = time.perf_counter()
        ops += wl["formula"](rows)
        t += time.perf_counter() - t0
        reps += 1
    return {
        "value": round(ops / t / 1e9, 3),
        "unit": "G dist-ops/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"dense torch formula (the reference's use_custom_cuda_func=False arithmetic) on {rows} of "
                  f"{wl['full_rows']} rows of the same workload, {reps} pass(es), {t:.1f} s",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The GPU's clock takes some tens of milliseconds of load to settle (--settle-ms covers that
    # for any --warmup); the defaults below are long enough for a stable mean.
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed set-up: run the workload this long before the warm-up steps so the clock settles")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="c1")
    ap.add_argument("--p", type=float, default=None,
                    help="exponent for --workload c2 or c4p (default 8, the configuration; the reference anneals it "
                         "to 1000)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true",
                    help="skip the comparison with the CPU oracle that runs before the timed region (profiler runs)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three plain 256 MiB device copies, the known-size kernel that "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.p is not None:
        if args.workload not in ("c2", "c4p") or not (args.p > 1 and math.isfinite(args.p)):
            sys.exit("--p applies to --workload c2 or c4p and must be a finite exponent above 1")
        global C2_P, C4_P
        C2_P = C4_P = args.p
    wl = WORKLOADS[args.workload](pkg, torch, dev)
    step = wl["step"]
    kname, flops_of, accept, kdesc, flops_per_op = wl["kernel"]

    # Parity first, in this process, on this workload's own tensors: a wrong result must not be timed.
    parity = {"checked": False, "note": "skipped (--no-parity)"}
    if not args.no_parity:
        import oracle
        from oracle import stack_check
        t0 = time.perf_counter()
        rep = wl["check"](oracle, stack_check)
        parity = rep.as_json()
        parity["seconds"] = round(time.perf_counter() - t0, 1)
        if not rep.ok:
            print(json.dumps({"parity": parity}))
            sys.exit("bench.py: the GPU results differ from the CPU oracle; nothing was timed")

    with KernelTimer(pkg.norm_dist_cpp, torch, kname, flops_of, accept) as kt:
        # Set-up, before the warm-up proper: keep the GPU under this load until its clock has settled
        # (after an idle period the first tens of milliseconds run 5-10 % slow), whatever --warmup says.
        if args.settle_ms > 0:
            step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            step()
            torch.cuda.synchronize()
            one = max(time.perf_counter() - t0, 1e-5)
            for _ in range(min(5000, int(args.settle_ms * 1e-3 / one) + 1)):   # back to back, no gaps
                step()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        kt.enabled = True
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        n_launch, k_ms, k_flops = kt.summary()

    if args.copy_probe:
        src = torch.empty(64 * 1024 * 1024, device=dev).uniform_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    ms_per_step = elapsed * 1e3 / args.steps
    ops = wl["ops"]
    value = ops / (ms_per_step * 1e-3) / 1e9
    achieved = k_flops / (k_ms * 1e-3) / 1e12 if k_ms > 0 else 0.0
    out = {
        "metric": "dist-neuron fwd+bwd G-ops/s, % FP32 VALU peak; img/s CIFAR 5120-wide net",
        "value": round(value, 2),
        "unit": "G dist-ops/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": wl["name"], "dist_ops_per_step": ops, **wl.get("routes", {}),
                   **({"routes": wl["layer_routes"]()} if "layer_routes" in wl else {})},
        "img_per_s": round(wl["images"] / (ms_per_step * 1e-3), 1),
        "pct_fp32_valu_peak": round(100 * value * 1e9 * flops_per_op / (FP32_PEAK_TFLOPS * 1e12), 2),
        "parity": parity,
        "roofline": {
            "bound": "valu",
            # the bench contract names "hbm" and "mfma"; this kernel's compute roof is neither: it is the fp32 vector ALU
            "bound_note": "compute roof, fp32 vector ALU (published dense fp32 peak); a max / power-sum reduction has "
                          "no multiply-accumulate, so there is no MFMA work on this path",
            "kernel": kdesc,
            "achieved": round(achieved, 2),
            "peak": FP32_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / FP32_PEAK_TFLOPS, 4),
            "dist_ops_per_s_T": round(achieved / flops_per_op, 3),
            "launches_timed": n_launch,
            "avg_launch_ms": round(k_ms, 4),
            "avg_flops_per_launch": k_flops,
            "traffic": None,
        },
    }
    # HBM bytes per launch of the roofline kernel (c1: average over the step's four tiled forward launches), from
    # two rocprofv3 --pmc runs of this command: FETCH_SIZE and WRITE_SIZE, each scaled by what the counter reads for
    # a plain copy of known size.  The figure is read from the counter summary kept under profiles/, which names
    # the kernel it was measured on; null when there is no summary for this workload's kernel.
    out["roofline"]["traffic"], out["roofline"]["traffic_source"] = profile_traffic(args.workload)
    for label, alt in wl.get("step_alt", []):
        for _ in range(args.warmup):
            alt()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            alt()
        torch.cuda.synchronize()
        out[label] = round((time.perf_counter() - t0) * 1e3 / args.steps, 4)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl)
        out["cpu_reference_formula"] = cpu_formula_baseline(wl)
    print(json.dumps(out))


# workload -> (counter summary under profiles/, the roofline kernel's name in it)
def traffic_profiles():
    c2_fused = C2_P != 2.0
    return {"c1": ("counters_c1_mlp_inf.md", "inf_forward_kernel"), "c1t": ("counters_c1t_training_step.md", "inf_forward_kernel"),
            "c0": ("counters_c0_fc_layer.md", "inf_forward_kernel"),
            "c2": (f"counters_c2_mlp_p{C2_P:g}.md", "norm_backward_fused_kernel" if c2_fused else "norm_backward_input_tiled_kernel"),
            "c3": ("counters_c3_certification.md", "bound_forward_kernel"),
            "c4": ("counters_c4_conv_columns.md", "inf_forward_shortk_kernel"),
            "c4i": ("counters_c4_conv_from_image.md", "inf_conv_forward_kernel"),
            "c4p": (f"counters_c4p_conv_p{C4_P:g}_from_image.md", "norm_conv_backward_kernel")}


def profile_traffic(workload):
    """(bytes per launch, source file) from the line 'traffic_bytes_per_launch[<kernel>]: <number>' of the
    workload's counter summary under profiles/, or (None, None)."""
    import re
    name, kernel = traffic_profiles().get(workload, (None, None))
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return None, None
    m = re.search(r"^traffic_bytes_per_launch\[" + re.escape(kernel) + r"\]:\s*([0-9.eE+]+)", open(path).read(), re.M)
    return (float(m.group(1)), "profiles/" + name) if m else (None, None)


if __name__ == "__main__":
    main()
