"""The two tolerances of the parity checks -- TEST INFRASTRUCTURE ONLY (tests/, bench.py's parity leg).

Defined here once; tests/helpers.py and oracle/stack_check.py import them.

* `plain_ratio`: |got - exact| <= atol + rtol * |exact| with rtol 1e-5 and atol 1e-6, the tolerance the task states.
  It applies to the p-norm forward and to every L_inf scatter gradient (the library sums those in double and rounds
  once, so they are the correctly rounded sums).
* `pnorm_grad_ratio`: the p-norm gradients only.  Such a gradient is a float32 sum of signed terms u^(p-1), u known
  to about 2e-7 relative, so each term is good to (p-1) * 2e-7 and the sum to that times sum|terms|, for any
  implementation (the reference's __powf and float atomics included).  Bound:
      s * (rtol * |exact| + atol * max(1, sum|terms|)),   s = max(1, p / 8).
  This is wider than the stated tolerance wherever sum|terms| > 1 or p > 8; the test run prints, per exponent, how far
  beyond the plain tolerance the worst element lies.
"""
RTOL = 1e-5
ATOL = 1e-6


def plain_ratio(got, exact, rtol=RTOL, atol=ATOL):
    """Worst |got - exact| / (atol + rtol * |exact|); <= 1 passes."""
    if got.numel() == 0:
        return 0.0
    err = (got.double() - exact.double()).abs()
    return float((err / (atol + rtol * exact.double().abs())).max())


def pnorm_grad_bound(exact, abs_terms, p, rtol=RTOL, atol=ATOL):
    scale = max(1.0, p / 8.0)
    return scale * (rtol * exact.double().abs() + atol * abs_terms.double().clamp_min(1.0))


def pnorm_grad_ratio(got, exact, abs_terms, p, rtol=RTOL, atol=ATOL):
    """Worst |got - exact| / pnorm_grad_bound; <= 1 passes."""
    if got.numel() == 0:
        return 0.0
    err = (got.double() - exact.double()).abs()
    return float((err / pnorm_grad_bound(exact, abs_terms, p, rtol, atol)).max())
