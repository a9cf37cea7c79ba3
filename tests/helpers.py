"""Closed forms used to pin the oracle and seeded input makers shared by the tests.

Nothing here calls the oracle's operators or the HIP library: these are independent
restatements of the mathematics in plain torch broadcasting.  The two assert_* helpers at
the end apply the tolerances defined once in oracle/tolerance.py.
"""
import torch

SIGN = -2147483648  # int32 with only bit 31 set


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def make_inputs(B, CO, CI, G, HW, seed=0, quantize=None):
    """x ~ U[0,1], w ~ N(0,1)/sqrt(K).  quantize=q rounds both to multiples of 1/q (forces ties)."""
    g = gen(seed)
    K = CI // G
    x = torch.rand(B, CI, HW, generator=g)
    w = torch.randn(CO, K, generator=g) / K ** 0.5
    if quantize:
        x = torch.round(x * quantize) / quantize
        w = torch.round(w * quantize) / quantize
    return x.contiguous(), w.contiguous()


def dense_diff(x, w, G):
    """(B, G, NG, K, HW) tensor of x - w in the reference layout."""
    B, CI, HW = x.shape
    CO, K = w.shape
    return x.reshape(B, G, 1, K, HW) - w.reshape(G, CO // G, K, 1)


def closed_inf_forward(x, w, G):
    """Values, first-maximum index and sign flag by torch broadcasting (fp32: sub/abs/max are exact)."""
    B, CI, HW = x.shape
    CO = w.shape[0]
    d = dense_diff(x, w, G)
    a = d.abs()
    val, idx = a.max(dim=3)  # CPU torch.max returns the first maximal index
    sign = torch.gather(d, 3, idx.unsqueeze(3)).squeeze(3) < 0
    pos = idx.to(torch.int32)
    pos = torch.where(sign, pos | SIGN, pos)
    pos = torch.where(val > 0, pos, torch.zeros_like(pos))  # nothing exceeds the initial 0
    return val.reshape(B, CO, HW), pos.reshape(B, CO, HW)


def closed_bound(lower, upper, w, G):
    B, CI, HW = lower.shape
    CO = w.shape[0]
    tl = dense_diff(lower, w, G)
    tu = dense_diff(upper, w, G)
    al, au = tl.abs(), tu.abs()
    up = torch.maximum(al, au).amax(dim=3)
    lo = torch.minimum(al, au)
    lo = torch.where((tl < 0) & (tu > 0), torch.zeros_like(lo), lo).amax(dim=3)
    return lo.reshape(B, CO, HW), up.reshape(B, CO, HW)


def closed_pnorm(x, w, G, p):
    """(sum |x-w|^p)^(1/p) in float64, max-normalised so it cannot overflow."""
    B, CI, HW = x.shape
    CO = w.shape[0]
    a = dense_diff(x.double(), w.double(), G).abs()
    m = a.amax(dim=3, keepdim=True).clamp_min(1e-300)
    out = ((a / m) ** p).sum(dim=3, keepdim=True) ** (1.0 / p) * m
    return out.reshape(B, CO, HW)


def unpack_pos(pos):
    idx = (pos & 0x7FFFFFFF).long()
    neg = pos < 0
    return idx, neg


def dense_inf_backward(grad_out, pos, CI, G):
    """One-hot expansion of the argmax-routed scatter in float64.
    Returns grad_x (B, CI, HW) and grad_w (CO, K)."""
    B, CO, HW = grad_out.shape
    K, NG = CI // G, CO // G
    idx, neg = unpack_pos(pos)
    g = grad_out.double()
    sg = torch.where(neg, -g, g)  # d out / d x = sign(x - w)
    onehot = torch.zeros(B, G, NG, K, HW, dtype=torch.float64)
    onehot.scatter_(3, idx.reshape(B, G, NG, 1, HW), sg.reshape(B, G, NG, 1, HW))
    grad_x = onehot.sum(dim=2).reshape(B, CI, HW)
    grad_w = -onehot.sum(dim=(0, 4)).reshape(CO, K)
    return grad_x, grad_w


# Worst err / bound seen by the gradient comparisons, per exponent (None: the L_inf scatter sums).  The test session
# prints it at the end (tests/conftest.py).
SUM_CLOSE_MARGINS = {}


def _record(p, worst, plain):
    seen = SUM_CLOSE_MARGINS.setdefault(p, {"calls": 0, "worst_err_over_bound": 0.0, "worst_err_over_plain_1e-5_1e-6": 0.0})
    seen["calls"] += 1
    seen["worst_err_over_bound"] = max(seen["worst_err_over_bound"], worst)
    seen["worst_err_over_plain_1e-5_1e-6"] = max(seen["worst_err_over_plain_1e-5_1e-6"], plain)


def assert_scatter_close(got, exact, rtol=None, atol=None):
    """An L_inf scatter gradient against the oracle's: the plain tolerance |got - exact| <= 1e-6 + 1e-5 * |exact|
    (oracle/tolerance.py:plain_ratio), whatever the number of terms on an element."""
    from oracle import tolerance
    worst = tolerance.plain_ratio(got, exact, rtol or tolerance.RTOL, atol or tolerance.ATOL)
    _record(None, worst, worst)
    assert worst <= 1.0, f"L_inf scatter: worst error is {worst:.3f} x the tolerance (rel 1e-5 / abs 1e-6)"
    return worst


def assert_sum_close(got, exact, abs_terms, p, rtol=None, atol=None):
    """A p-norm gradient (a float32 sum of signed terms) against its exact value, with the tolerance of
    oracle/tolerance.py:pnorm_grad_ratio, which scales with sum|terms| and max(1, p/8).
    Returns the worst err / bound ratio (<= 1) and records it per exponent."""
    from oracle import tolerance
    assert p is not None, "L_inf scatters are compared with assert_scatter_close"
    rtol, atol = rtol or tolerance.RTOL, atol or tolerance.ATOL
    worst = tolerance.pnorm_grad_ratio(got, exact, abs_terms, p, rtol, atol)
    _record(p, worst, tolerance.plain_ratio(got, exact, rtol, atol))
    assert worst <= 1.0, f"p = {p}: worst error is {worst:.3f} x the float32-sum tolerance"
    return worst
