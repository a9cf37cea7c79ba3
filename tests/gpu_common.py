"""Helpers for the GPU parity tests: every call goes through the C ABI (ctypes binding)."""
import sys

import torch

import __graft_entry__ as entry

pkg = entry.load_package()
cpp = pkg.norm_dist_cpp
DEV = torch.device("cuda:0")


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def set_tile(choice):
    rc = pkg._lib.lib().ldist_set_tile_override(choice)
    assert rc == 0


def gpu_inf_forward(x, w, G):
    xd, wd = x.to(DEV), w.to(DEV)
    out = torch.empty(x.size(0), w.size(0), x.size(2), device=DEV)
    pos = torch.empty(x.size(0), w.size(0), x.size(2), device=DEV, dtype=torch.int32)
    cpp.inf_dist_forward(xd, wd, out, pos, G)
    torch.cuda.synchronize()
    return out.cpu(), pos.cpu()


def gpu_bound_forward(lo, up, w, G):
    out_l = torch.empty(lo.size(0), w.size(0), lo.size(2), device=DEV)
    out_u = torch.empty_like(out_l)
    cpp.inf_dist_bound_forward(lo.to(DEV), up.to(DEV), w.to(DEV), out_l, out_u, G)
    torch.cuda.synchronize()
    return out_l.cpu(), out_u.cpu()


def gpu_norm_forward(x, w, G, p):
    out = torch.empty(x.size(0), w.size(0), x.size(2), device=DEV)
    cpp.norm_dist_forward(x.to(DEV), w.to(DEV), out, G, p)
    torch.cuda.synchronize()
    return out.cpu()


def gpu_value_bound_forward(x, lo, up, w, G, mean=None, bias=None):
    out = torch.full((x.size(0), w.size(0), x.size(2)), float("nan"), device=DEV)
    out_l, out_u = torch.full_like(out, float("nan")), torch.full_like(out, float("nan"))
    cpp.inf_dist_value_bound_forward(x.to(DEV), lo.to(DEV), up.to(DEV), w.to(DEV), out, out_l, out_u, G,
                                     None if mean is None else mean.to(DEV), None if bias is None else bias.to(DEV))
    torch.cuda.synchronize()
    return out.cpu(), out_l.cpu(), out_u.cpu()
