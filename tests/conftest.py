import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_count():
    import torch
    return torch.cuda.device_count()


def pytest_collection_modifyitems(config, items):
    if _gpu_count() > 0:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """How much of the float32-sum tolerance the gradient comparisons used, per exponent p."""
    try:
        from helpers import SUM_CLOSE_MARGINS
    except ImportError:
        return
    if not SUM_CLOSE_MARGINS:
        return
    terminalreporter.write_sep("-", "assert_sum_close: worst error / tolerance per exponent")
    for p in sorted(SUM_CLOSE_MARGINS, key=lambda v: (v is not None, v or 0)):
        m = SUM_CLOSE_MARGINS[p]
        label = "L_inf scatter" if p is None else f"p = {p:g}"
        terminalreporter.write_line(
            f"{label:>14}: {m['calls']:5d} comparisons, worst err/bound {m['worst_err_over_bound']:.3f}; against plain "
            f"rel 1e-5 / abs 1e-6 the worst is {m['worst_err_over_plain_1e-5_1e-6']:.2f} x")
