"""The C-ABI library loads on a machine without a GPU, exports every symbol that
include/ldist.h declares, and rejects bad arguments before touching a device."""
import ctypes
import os
import re

import pytest

import __graft_entry__ as entry

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    pkg = entry.load_package()
    if not os.path.exists(pkg.LIB_PATH):
        pkg.build_library()
    return pkg._lib.lib()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ldist.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ldist_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_seven_reference_entry_points():
    names = declared_symbols()
    for ref in ("norm_dist_forward", "norm_dist_backward_input", "norm_dist_backward_weight", "inf_dist_forward",
                "inf_dist_bound_forward", "inf_dist_backward_input", "inf_dist_backward_weight"):
        assert "ldist_" + ref in names  # reference model/norm_dist.cpp:92-100


def test_every_declared_symbol_is_exported(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_binding_signatures_cover_all_compute_entry_points():
    pkg = entry.load_package()
    compute = [n for n in declared_symbols() if "_dist_" in n or n in ("ldist_mean_shift", "ldist_adamw_lp_step", "ldist_unfold", "ldist_fold")]
    assert sorted(pkg._lib.SIGNATURES) == sorted(compute)


def test_version_and_error_strings(lib):
    assert lib.ldist_version() == 100
    for code in (0, -1, -2, -3, -4, -5, -99):
        assert isinstance(lib.ldist_strerror(code), bytes) and lib.ldist_strerror(code)
    assert lib.ldist_set_tile_override(7) == -1 and lib.ldist_set_tile_override(4) == 0 and lib.ldist_set_tile_override(-1) == 0


def test_argument_checks_need_no_device(lib):
    one = ctypes.c_void_p(16)  # never dereferenced: the size checks fail first
    assert lib.ldist_inf_dist_forward(None, one, 1, 1, 1, 1, 1, one, one, None) == -1
    assert lib.ldist_inf_dist_forward(one, one, 0, 1, 1, 1, 1, one, one, None) == -1
    assert lib.ldist_inf_dist_forward(one, one, 2, 4, 6, 4, 1, one, one, None) == -1      # CI % G
    assert lib.ldist_inf_dist_forward(one, one, 2, 6, 4, 4, 1, one, one, None) == -1      # CO % G
    assert lib.ldist_inf_dist_forward(one, one, 1 << 20, 1 << 12, 8, 1, 1, one, one, None) == -2  # 2^32 outputs
    assert lib.ldist_norm_dist_forward(one, one, 1, 1, 1, 1, 1, one, 1.0, None) == -1     # p must exceed 1
    assert lib.ldist_norm_dist_forward(one, one, 1, 1, 1, 1, 1, one, float("inf"), None) == -1
    assert lib.ldist_norm_dist_backward_weight(one, one, one, one, 1, 1, 1, 1, 1, None, 8.0, None) == -1
    assert lib.ldist_inf_dist_bound_forward(one, None, one, 1, 1, 1, 1, 1, one, one, None) == -1
    assert lib.ldist_inf_dist_backward_input_overwrite(one, one, 1, 1, 1, 1, 0, one, None) == -1
    assert lib.ldist_inf_dist_value_bound_forward(one, one, None, one, 1, 1, 1, 1, 1, None, None, one, one, one, None) == -1
    assert lib.ldist_inf_dist_value_bound_forward(one, one, one, one, 1, 3, 4, 2, 1, None, None, one, one, one, None) == -1


def test_conv_forward_geometry_query_needs_no_device(lib):
    ok = lib.ldist_inf_dist_conv_forward_supported
    assert ok(128, 32, 32, 128, 4, 3, 3, 1, 1, 1) == 1      # the benchmark layer
    assert ok(3, 32, 32, 96, 1, 3, 3, 1, 1, 1) == 1         # the CIFAR conv net's first layer
    assert ok(16, 32, 32, 64, 1, 3, 3, 2, 1, 1) == 1        # a stride-2 layer
    assert ok(96, 32, 32, 96, 1, 3, 3, 1, 1, 1) == 1        # 96 channels in one group: staged four at a time
    assert ok(96, 32, 32, 192, 1, 3, 3, 2, 1, 1) == 1       # the CIFAR conv net's stride-2 layer
    assert ok(90, 32, 32, 96, 1, 3, 3, 1, 1, 1) == 0        # too many channels to stay in LDS, and not a multiple of four
    assert ok(16, 28, 28, 32, 1, 3, 3, 1, 1, 1) == 1        # output width 28: the last segment of a row is partly idle
    assert ok(4, 16, 16, 8, 1, 5, 5, 1, 2, 1) == 0          # window
    assert ok(4, 16, 16, 8, 1, 3, 3, 1, 2, 2) == 0          # dilation
    assert ok(4, 16, 16, 8, 3, 3, 3, 1, 1, 1) == 0          # channels do not divide into the groups
    one = ctypes.c_void_p(16)
    assert lib.ldist_inf_dist_conv_forward(one, one, 1, 4, 28, 28, 8, 1, 5, 5, 1, 2, 1, one, one, None) == -5
    assert lib.ldist_inf_dist_conv_forward(None, one, 1, 4, 32, 32, 8, 1, 3, 3, 1, 1, 1, one, one, None) == -1
    okb = lib.ldist_inf_dist_bound_conv_forward_supported
    assert okb(128, 32, 32, 128, 4, 3, 3, 1, 1, 1) == 1 and okb(90, 32, 32, 96, 1, 3, 3, 1, 1, 1) == 1   # any channel count
    assert okb(16, 28, 28, 32, 1, 3, 3, 1, 1, 1) == 1 and okb(4, 16, 16, 8, 1, 5, 5, 1, 2, 1) == 0
    assert lib.ldist_inf_dist_bound_conv_forward(one, one, one, 1, 4, 28, 28, 8, 1, 5, 5, 1, 2, 1, one, one, None) == -5
    assert lib.ldist_inf_dist_bound_conv_forward(one, None, one, 1, 4, 32, 32, 8, 1, 3, 3, 1, 1, 1, one, one, None) == -1
    assert lib.ldist_set_conv_rows_override(-1) == -1 and lib.ldist_set_conv_rows_override(0) == 0
    assert lib.ldist_set_conv_staging_override(4) == -1 and lib.ldist_set_conv_staging_override(0) == 0
