"""Whole-stack parity of the fully connected distance net against the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Used by tests/ and by bench.py's parity leg (which runs before the timed region).  Nothing in the product
package imports this module.

The net under test is driven through its own forward / backward once, with hooks that record what every layer
really received and produced on the GPU; the oracle then repeats every layer on exactly those inputs
("teacher forced"), so each comparison is as sharp as the operator allows:

* L_inf values: bit-exact (fp32 sub / abs / max are exact and order-independent);
* arg-max indices with their sign bits: bit-exact, from the caller's `inf_forward` (the library's forward entry point
  run again on the recorded input: the same launch the layer made, whose values must equal the recorded ones bit
  for bit), and once more through both scatter gradients, which move if a single index or sign differs;
* L_inf scatter gradients: rel 1e-5 / abs 1e-6 (the library rounds double sums once);
* p-norm values: rel 1e-5 / abs 1e-6; gradients: the float32-sum tolerance of `sum_ratio` (ratio <= 1 passes);
* the mean shift: abs 2e-6 against the float64 mean, or four units in the last place of the largest input where that
  is more (a float32 difference of numbers of size X cannot be closer than ulp(X); outputs grow past 16 only at
  exponents below the reference's schedule, p < 8 on 5120 inputs);
* and, free running from the input (the oracle feeding itself), the last layer's output: every layer is
  1-Lipschitz in the L_inf norm, so rounding of the shifts cannot grow on the way.

Reference arithmetic: model/inf_dist_cuda.cu:10-171, model/norm_dist_cuda.cu:228-425 (operators),
model/norm_dist.py:85-96 (mean shift), model/mlp.py:17-23 (stack), model/bound_module.py:95-103 (margins).
"""
import math

import torch

from . import (inf_dist_backward_input, inf_dist_backward_weight, inf_dist_bound_forward, inf_dist_forward, mean_shift,
               norm_dist_backward_input, norm_dist_backward_weight, norm_dist_forward)


from .tolerance import plain_ratio, pnorm_grad_ratio


def sum_ratio(got, exact, abs_terms, p):
    """A p-norm gradient against the oracle's: worst error / bound with the float32-sum tolerance
    (oracle/tolerance.py:pnorm_grad_ratio)."""
    return pnorm_grad_ratio(got, exact, abs_terms, p)


def close_ratio(got, exact, rtol=1e-5, atol=1e-6):
    """Worst |got - exact| / (atol + rtol*|exact|): the plain tolerance, also for every L_inf scatter gradient."""
    return plain_ratio(got, exact, rtol, atol)


class Report:
    """Collects comparisons; `ok` stays true while exact ones are equal and every ratio is <= 1."""

    def __init__(self):
        self.ok = True
        self.exact = 0            # tensors compared bit for bit
        self.toleranced = 0       # tensors compared within a tolerance
        self.worst_ratio = 0.0    # largest err / bound of the toleranced ones
        self.max_rel_err = 0.0    # largest max|got - exact| / max|exact| over all compared tensors
        self.failures = []

    def _rel(self, got, exact):
        scale = float(exact.double().abs().max())
        if scale > 0:
            self.max_rel_err = max(self.max_rel_err, float((got.double() - exact.double()).abs().max()) / scale)

    def equal(self, what, got, exact):
        self.exact += 1
        self._rel(got, exact)
        if not torch.equal(got, exact):
            self.ok = False
            self.failures.append(f"{what}: {int((got != exact).sum())} of {got.numel()} elements differ")

    def ratio(self, what, r, got=None, exact=None):
        self.toleranced += 1
        if got is not None:
            self._rel(got, exact)
        self.worst_ratio = max(self.worst_ratio, r)
        if not r <= 1.0:
            self.ok = False
            self.failures.append(f"{what}: error is {r:.3g} x the tolerance")

    def as_json(self):
        return {"checked": self.ok, "max_rel_err": self.max_rel_err, "worst_err_over_tolerance": round(self.worst_ratio, 4),
                "tensors_bit_exact": self.exact, "tensors_within_tolerance": self.toleranced, "failures": self.failures[:8]}


def _layers(model):
    return list(model.fc) + [model.fc_last]


def record_training_step(model, x_dev, upstream_dev):
    """One forward + backward of `model` (an MLP of this package, training mode) with hooks; returns per layer
    a dict of CPU tensors: input, raw (operator output before the shift), shifted (after shift and bias),
    grad_raw (gradient arriving at the operator output), grad_input, grad_weight."""
    rec = [dict() for _ in _layers(model)]
    handles = []

    def pre(i):
        def hook(mod, args):
            t = args[0]
            rec[i]["input"] = t.detach()
            if t.requires_grad:
                t.register_hook(lambda g, i=i: rec[i].__setitem__("grad_input", g.detach()))
        return hook

    def norm_hook(i):
        def hook(mod, args, out):
            raw = args[0]
            rec[i]["raw"] = raw.detach()
            raw.register_hook(lambda g, i=i: rec[i].__setitem__("grad_raw", g.detach()))
        return hook

    def post(i):
        def hook(mod, args, out):
            rec[i]["shifted"] = out[0].detach()
            if mod.normalize is None:      # no shift module to hook: the operator output is out - bias
                raw = out[0] if mod.bias is None else None
                rec[i]["raw"] = None if raw is None else raw.detach()
        return hook

    for i, layer in enumerate(_layers(model)):
        handles.append(layer.register_forward_pre_hook(pre(i)))
        handles.append(layer.register_forward_hook(post(i)))
        if layer.normalize is not None:
            handles.append(layer.normalize.register_forward_hook(norm_hook(i)))
    try:
        for prm in model.parameters():
            prm.grad = None
        x_dev = x_dev.detach().requires_grad_(True)
        y, _, _ = model(x_dev)
        y.backward(upstream_dev)
        if x_dev.is_cuda:
            torch.cuda.synchronize()
    finally:
        for h in handles:
            h.remove()
    out = []
    for r, layer in zip(rec, _layers(model)):
        d = {k: (None if v is None else v.float().cpu().reshape(v.size(0), -1, 1).contiguous()) for k, v in r.items()}
        d["grad_weight"] = layer.weight.grad.detach().cpu().reshape(layer.weight.size(0), -1).contiguous()
        d["weight"] = layer.weight.detach().cpu().reshape(layer.weight.size(0), -1).contiguous()
        d["bias"] = None if layer.bias is None else layer.bias.detach().cpu()
        d["has_shift"] = layer.normalize is not None
        out.append(d)
    return out, (-y).detach().cpu()     # the net negates its output (model/mlp.py:22)


def check_training_step(model, x_cpu, upstream_cpu, p, dev, rows=None, weight_rows=None, report=None, inf_forward=None):
    """Teacher-forced comparison of one training step of the MLP with the oracle.  `rows` (slice of the batch)
    and `weight_rows` (slice of each layer's outputs) bound the oracle's work for the p-norm operators; None
    means everything.  `inf_forward(x_cpu, w_cpu) -> (values, pos)` (CPU tensors) is the library's L_inf forward
    entry point, for the direct comparison of the indices at p = inf.  Returns the Report."""
    rep = report or Report()
    inf = math.isinf(p)
    layers, y_gpu = record_training_step(model, x_cpu.to(dev), upstream_cpu.to(dev))
    B = x_cpu.size(0)
    rs = rows or slice(0, B)
    h_free = x_cpu.reshape(B, -1, 1).contiguous()
    for i, L in enumerate(layers):
        w, xin = L["weight"], L["input"]
        CO, CI = w.shape
        ws = weight_rows if (weight_rows is not None and CO > (weight_rows.stop - weight_rows.start)) else slice(0, CO)
        name = f"layer {i} ({CI}->{CO})"
        raw = L["raw"]
        assert raw is not None, "every layer of the benchmark net has a mean shift"
        # forward of the operator on the GPU's own input
        if inf:
            ev, ep = inf_dist_forward(xin[rs].contiguous(), w, 1)
            rep.equal(name + " values", raw[rs], ev)
            if inf_forward is not None:
                gv, gp = inf_forward(xin[rs].contiguous(), w)
                rep.equal(name + " values of the repeated launch against the layer's own", gv, raw[rs])
                rep.equal(name + " arg-max indices and signs", gp, ep)
        else:
            ev = norm_dist_forward(xin[rs].contiguous(), w, 1, p)
            rep.ratio(name + " values", close_ratio(raw[rs], ev), raw[rs], ev)
        # the mean shift (training mode: batch mean) and the bias
        es, _ = mean_shift(raw)
        if L["bias"] is not None:
            es = es + L["bias"].view(1, -1, 1)
        ms_atol = max(2e-6, 4 * 2.0 ** -23 * float(raw.abs().max()))
        rep.ratio(name + " mean shift", close_ratio(L["shifted"], es, rtol=1e-6, atol=ms_atol), L["shifted"], es)
        # backward: the gradient that reached the operator output on the GPU goes through the oracle
        g = L["grad_raw"]
        if inf:
            ev_all, ep_all = (ev, ep) if rs == slice(0, B) else inf_dist_forward(xin, w, 1)
            egw = inf_dist_backward_weight(g, ep_all, CI, 1)
            rep.ratio(name + " grad_weight", close_ratio(L["grad_weight"], egw), L["grad_weight"], egw)
            if L.get("grad_input") is not None:
                egx = inf_dist_backward_input(g, ep_all, CI, 1)
                rep.ratio(name + " grad_input", close_ratio(L["grad_input"], egx), L["grad_input"], egx)
        else:
            gw_s = slice(ws.start, ws.stop)
            egw, mgw = norm_dist_backward_weight(g[:, gw_s].contiguous(), xin, w[gw_s].contiguous(),
                                                 raw[:, gw_s].contiguous(), 1, p, with_abs_terms=True)
            rep.ratio(name + " grad_weight", sum_ratio(L["grad_weight"][gw_s], egw, mgw, p), L["grad_weight"][gw_s], egw)
            if L.get("grad_input") is not None:
                egx, mgx = norm_dist_backward_input(g[rs].contiguous(), xin[rs].contiguous(), w, raw[rs].contiguous(), 1, p,
                                                    with_abs_terms=True)
                rep.ratio(name + " grad_input", sum_ratio(L["grad_input"][rs], egx, mgx, p), L["grad_input"][rs], egx)
        # free-running oracle stack (full batch only: the shift needs every row)
        if h_free is not None and rs == slice(0, B) and inf:
            fv, _ = inf_dist_forward(h_free, w, 1)
            h_free, _ = mean_shift(fv)
            if L["bias"] is not None:
                h_free = (h_free + L["bias"].view(1, -1, 1)).contiguous()
        else:
            h_free = None
    if h_free is not None:
        rep.ratio("free-running oracle stack, last output", close_ratio(y_gpu.reshape(B, -1, 1), h_free, rtol=0, atol=1e-4),
                  y_gpu.reshape(B, -1, 1), h_free)
    return rep


def oracle_certification(ws, means, biases, x, lo, up, targets):
    """The oracle's evaluation-mode pass of the stack with interval bounds and the final margins:
    per layer value / lower / upper minus the running mean (plus bias), negated at the end with lower and upper
    exchanged (model/mlp.py:22-23), then margins res[b, j] = upper'[b, j] - lower'[b, t_b], res[b, t_b] = 0
    (model/bound_module.py:95-103)."""
    B = x.size(0)
    h, l, u = (t.reshape(B, -1, 1).contiguous() for t in (x, lo, up))
    for w, m, b in zip(ws, means, biases):
        out, _ = inf_dist_forward(h, w, 1)
        ol, ou = inf_dist_bound_forward(l, u, w, 1)
        outs = []
        for t in (out, ol, ou):
            if m is not None:
                t = t - m.view(1, -1, 1)
            if b is not None:
                t = t + b.view(1, -1, 1)
            outs.append(t.contiguous())
        h, l, u = outs
    y, lower, upper = (-h).squeeze(-1), (-u).squeeze(-1), (-l).squeeze(-1)
    res = upper - torch.gather(lower, 1, targets.view(-1, 1))
    res = res.scatter(1, targets.view(-1, 1), 0.0)
    return y, lower, upper, res
