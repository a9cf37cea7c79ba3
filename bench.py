#!/usr/bin/env python3
"""Benchmark of the distance-neuron hot path on one MI355X.

Workload (BASELINE.json configs[1]): the CIFAR-10-shaped 5-layer L_inf-dist MLP
3072 -> 5120 -> 5120 -> 5120 -> 5120 -> 10 at p = inf, batch 512, fp32, forward
plus backward (grad_x of every layer and every grad_w).  A "step" is one
forward+backward pass over one synthetic batch that already sits in HBM.

Prints ONE JSON line.  `value` is G dist-ops/s, a dist-op being one (row, output,
input) triple of a forward pass (48.35 G per step).  `roofline` is measured live
on the dominant kernel (the tiled L_inf forward) with events on the stream the
kernels run on; `cpu_baseline` times the CPU oracle on a bounded row sample of
the same workload.
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
BATCH = 512
CIFAR_MEAN = (0.4914, 0.4822, 0.4465)
CIFAR_STD = 0.2009
FP32_PEAK_TFLOPS = 157.3          # MI355X vector fp32 (packed FMA) peak
VALU_ISSUE_PEAK_T = 39.3          # 256 CU x 64 lanes x 2.4 GHz lane-instructions per second
FLOPS_PER_DIST_OP = 2             # sub, max; abs/compare/index bookkeeping count as zero


def dist_ops_per_forward(batch):
    return sum(batch * a * b for a, b in zip(LAYERS[:-1], LAYERS[1:]))


def make_inputs(batch, seed=0):
    import torch
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(batch, 3, 32, 32, generator=g)
    mean = torch.tensor(CIFAR_MEAN).view(1, 3, 1, 1)
    x = ((x - mean) / CIFAR_STD).reshape(batch, -1).contiguous()
    ws = [torch.randn(o, i, generator=g) / math.sqrt(i) for i, o in zip(LAYERS[:-1], LAYERS[1:])]
    upstream = torch.randn(batch, LAYERS[-1], generator=g)
    return x, ws, upstream


def build_model(pkg, ws, dev):
    import torch
    model = pkg.MLP(depth=5, width=5, input_dim=3072, num_classes=10, head_mean_normalize=True)
    with torch.no_grad():
        for layer, w in zip(list(model.fc) + [model.fc_last], ws):
            layer.weight.copy_(w.view_as(layer.weight))
    pkg.set_p_norm(model, float("inf"))
    return model.to(dev).train()


class KernelTimer:
    """Brackets every tiled L_inf forward launch with events on the current stream."""

    def __init__(self, cpp, torch):
        self.cpp, self.torch = cpp, torch
        self.orig = cpp.inf_dist_forward
        self.records = []
        self.enabled = False

    def __enter__(self):
        def timed(input, weight, output, pos, G):
            if not self.enabled or weight.size(0) // G <= 16:   # the 10-way head runs a different kernel
                return self.orig(input, weight, output, pos, G)
            a = self.torch.cuda.Event(enable_timing=True)
            b = self.torch.cuda.Event(enable_timing=True)
            a.record()
            self.orig(input, weight, output, pos, G)
            b.record()
            flops = FLOPS_PER_DIST_OP * input.size(0) * input.size(2) * weight.size(0) * weight.size(1)
            self.records.append((a, b, flops))
        self.cpp.inf_dist_forward = timed
        return self

    def __exit__(self, *exc):
        self.cpp.inf_dist_forward = self.orig

    def summary(self):
        ms = sum(a.elapsed_time(b) for a, b, _ in self.records)
        flops = sum(f for _, _, f in self.records)
        n = len(self.records)
        return n, ms / max(n, 1), flops / max(n, 1)


def cpu_baseline(target_seconds=12.0):
    """C1 forward+backward with the CPU oracle (C, OpenMP) on a row subset sized to ~target_seconds."""
    import torch
    import oracle
    x, ws, upstream = make_inputs(BATCH)

    def run(rows):
        t0 = time.perf_counter()
        h = x[:rows].reshape(rows, -1, 1).contiguous()
        saved = []
        for w in ws:
            out, pos = oracle.inf_dist_forward(h, w, 1)
            saved.append((h.size(1), pos))
            h = (out - out.mean(dim=0, keepdim=True)).contiguous()
        g = upstream[:rows].reshape(rows, -1, 1).contiguous()
        for (ci, pos), w in zip(reversed(saved), reversed(ws)):
            g = (g - g.mean(dim=0, keepdim=True)).contiguous()
            oracle.inf_dist_backward_weight(g, pos, ci, 1)
            g = oracle.inf_dist_backward_input(g, pos, ci, 1)
        return time.perf_counter() - t0

    probe_rows = 8
    t = run(probe_rows)
    rows = int(max(probe_rows, min(BATCH, probe_rows * target_seconds / max(t, 1e-3))))
    t = run(rows)
    reps = 1
    while t < target_seconds and reps < 64:      # fast hosts: repeat the pass until the sample is long enough
        t += run(rows)
        reps += 1
    ops = dist_ops_per_forward(rows) * reps
    return {
        "value": round(ops / t / 1e9, 3),
        "unit": "G dist-ops/s",
        "cores": oracle.num_threads(),
        "kind": "port",
        "sample": f"C oracle (OpenMP), forward+backward of the same 5-layer stack on {rows} of {BATCH} rows, "
                  f"{reps} pass(es), {t:.1f} s",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
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

    x, ws, upstream = make_inputs(BATCH)
    model = build_model(pkg, ws, dev)
    xd = x.to(dev).requires_grad_(True)
    up = upstream.to(dev)

    def step():
        xd.grad = None
        for prm in model.parameters():
            prm.grad = None
        y, _, _ = model(xd)
        y.backward(up)

    with KernelTimer(pkg.norm_dist_cpp, torch) as kt:
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
    ops = dist_ops_per_forward(BATCH)
    value = ops / (ms_per_step * 1e-3) / 1e9
    achieved = k_flops / (k_ms * 1e-3) / 1e12 if k_ms > 0 else 0.0
    out = {
        "metric": "dist-neuron fwd+bwd G-ops/s, % FP32 VALU peak; img/s CIFAR 5120-wide net",
        "value": round(value, 2),
        "unit": "G dist-ops/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: 5-layer L_inf-dist MLP 3072-5120-5120-5120-5120-10, p=inf, batch 512, "
                               "forward+backward (all grad_x and grad_w), mean shift in training mode",
                   "batch": BATCH, "dist_ops_per_step": ops},
        "img_per_s": round(BATCH / (ms_per_step * 1e-3), 1),
        "pct_fp32_valu_peak": round(100 * value * 1e9 * FLOPS_PER_DIST_OP / (FP32_PEAK_TFLOPS * 1e12), 2),
        "roofline": {
            "bound": "mfma",
            "kernel": "inf_forward_kernel (tiled L_inf forward, VALU only: the max-plus reduction cannot use MFMA; "
                      "'mfma' here names the compute roof, priced at the fp32 vector peak)",
            "achieved": round(achieved, 2),
            "peak": FP32_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / FP32_PEAK_TFLOPS, 4),
            "frac_of_valu_issue_peak": round(achieved * 1e12 / FLOPS_PER_DIST_OP / (VALU_ISSUE_PEAK_T * 1e12), 4),
            "launches_timed": n_launch,
            "avg_launch_ms": round(k_ms, 4),
            "avg_flops_per_launch": k_flops,
            "traffic": None,
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
