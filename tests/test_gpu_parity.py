"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on the same seeded inputs.

Bars: L_inf forward values and indices and the interval bounds are bit-exact
(torch.equal); scatter gradients and everything p-norm are within rel 1e-5 /
abs 1e-6 of the oracle's double-precision result.
"""
import math

import pytest
import torch

import oracle
from helpers import SIGN, assert_scatter_close, assert_sum_close, gen, make_inputs

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6

# B, CO, CI, G, HW   -- fc and conv layouts, ragged sizes, groups, vector and scalar load paths
SHAPES = [
    (5, 7, 3, 1, 1),          # tiny, few outputs (one-wave-per-row kernel)
    (33, 100, 77, 1, 1),      # K % 4 != 0: scalar loads, ragged M / N / K
    (130, 70, 260, 1, 1),     # vector loads, M and N tails, K tail inside a chunk
    (20, 40, 12, 1, 1),       # vector loads with K shorter than one chunk of 32
    (9, 24, 36, 1, 1),        # vector loads, second chunk holds a single group of four
    (64, 96, 96, 3, 1),       # groups, K = 32 exactly one chunk
    (64, 48, 96, 3, 1),       # groups with 16 outputs each
    (256, 160, 784, 1, 1),    # MNIST-sized K, two N tiles of 80
    (512, 10, 640, 1, 1),     # classification head
    (2, 8, 12, 1, 16),        # conv layout, HW % 4 == 0
    (3, 6, 9, 3, 5),          # conv layout, scalar loads, groups
    (2, 64, 64, 2, 64),       # conv layout, 32 outputs per group
    (4, 128, 1152, 4, 100),   # the unfolded 3x3 conv layer shape at a small image
    (1, 40, 2000, 1, 36),     # conv layout, long K
]
TILES = [-1, 0, 1, 2, 3, 4]


@pytest.fixture(autouse=True)
def _reset_tile():
    from gpu_common import pkg, set_tile
    yield
    set_tile(-1)
    pkg._lib.lib().ldist_set_conv_rows_override(0)
    pkg._lib.lib().ldist_set_conv_staging_override(0)


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("quant", [None, 8])
def test_inf_forward_bit_exact(shape, tile, quant):
    from gpu_common import gpu_inf_forward, say, set_tile
    B, CO, CI, G, HW = shape
    say("inf_forward", shape, "tile", tile, "quant", quant)
    x, w = make_inputs(B, CO, CI, G, HW, seed=sum(shape), quantize=quant)
    set_tile(tile)
    out, pos = gpu_inf_forward(x, w, G)
    eo, ep = oracle.inf_dist_forward(x, w, G)
    assert torch.equal(out, eo)
    assert torch.equal(pos, ep)


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("shape", SHAPES + [(130, 170, 300, 1, 1), (70, 96, 1028, 2, 1), (512, 5120, 784, 1, 1)])
def test_inf_forward_values_only_matches_the_full_forward(shape, tile):
    """inf_dist_forward_values (no pos; what a forward without a gradient to follow calls) against the oracle's
    values, bit for bit, on every tiling; where it says it has no kernel (conv layout, 16 outputs per group or
    fewer, K not a multiple of four) it must leave the output alone."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = shape
    say("inf_forward values only", shape, "tile", tile)
    x, w = make_inputs(B, CO, CI, G, HW, seed=sum(shape) + 1)
    set_tile(tile)
    out = torch.full((B, CO, HW), -7.0, device=DEV)
    done = cpp.inf_dist_forward_values(x.to(DEV), w.to(DEV), out, G)
    assert done == (HW == 1 and CO // G > 16 and (CI // G) % 4 == 0)
    if done:
        assert torch.equal(out.cpu(), oracle.inf_dist_forward(x, w, G)[0])
    else:
        assert bool((out == -7.0).all())


def test_norm_dist_without_a_gradient_takes_the_values_only_forward():
    """norm_dist at p = inf: the same values with and without a gradient to follow (the second through the kernel
    without pos), and a gradient where one is asked for."""
    from gpu_common import DEV, pkg
    g = torch.Generator().manual_seed(5)
    x, w = torch.rand(96, 200, 1, generator=g).to(DEV), torch.rand(160, 200, generator=g).to(DEV)
    with torch.no_grad():
        y0 = pkg.norm_dist(x, w.clone().requires_grad_(), 1, float("inf"))
    wr = w.clone().requires_grad_()
    y1 = pkg.norm_dist(x, wr, 1, float("inf"))
    assert not y0.requires_grad and y1.requires_grad and torch.equal(y0, y1.detach())
    y1.sum().backward()
    assert wr.grad is not None and bool((wr.grad != 0).any())


# Shapes for the fully connected grad_weight kernels.  With at least 4 * 256 blocks of output rows the kernel with
# bins of one row runs (blocks of 4 rows up to batch 512, 3 up to 682, 2 up to 1024): (70, 4104, 36) and
# (300, 4096, 784) full blocks and 128-bit row stores; (70, 4102, 38) a ragged last block (4102 = 4 * 1025 + 2) and
# rows that are not a multiple of four (scalar stores); (600, 3100, 36) blocks of three rows with a ragged last one;
# (1000, 2050, 20) blocks of two; (16, 4104, 100, 2) two groups.  The others take the kernel with bins for a whole
# block, in one launch with grad_input ((33, 1600, 5120), (16, 2064, 100, 2)) or as two launches.
FC_SCATTER_SHAPES = [(70, 4104, 36, 1, 1), (300, 4096, 784, 1, 1), (70, 4102, 38, 1, 1), (600, 3100, 36, 1, 1),
                     (1000, 2050, 20, 1, 1), (16, 4104, 100, 2, 1), (33, 1600, 5120, 1, 1), (16, 2064, 100, 2, 1),
                     (40, 96, 64, 1, 1), (3, 24, 18, 3, 4)]


@pytest.mark.parametrize("shape", FC_SCATTER_SHAPES)
def test_inf_backward_both_gradients_in_one_call(shape):
    """inf_dist_backward_overwrite against the oracle: one launch whose workgroups do either scatter where the layer
    is fully connected with enough blocks of output rows to fill the device; the last two shapes fall back to the two
    kernels inside the call."""
    from gpu_common import DEV, cpp, say
    B, CO, CI, G, HW = shape
    say("inf_backward both", shape)
    x, w = make_inputs(B, CO, CI, G, HW, seed=sum(shape), quantize=8)   # quantised: ties and shared maxima
    _, ep = oracle.inf_dist_forward(x, w, G)
    go = torch.randn(B, CO, HW, generator=gen(77))
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.full((CO, CI // G), float("nan"), device=DEV)
    cpp.inf_dist_backward_overwrite(go.to(DEV), ep.to(DEV), gx, gw, G)
    torch.cuda.synchronize()
    assert_scatter_close(gx.cpu(), oracle.inf_dist_backward_input(go, ep, CI, G))
    assert_scatter_close(gw.cpu(), oracle.inf_dist_backward_weight(go, ep, CI, G))


@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("shape", FC_SCATTER_SHAPES)
def test_inf_backward_weight_alone(shape, accumulate):
    """grad_weight through its own entry points: the one that writes the gradient whole, on a buffer that starts as
    NaN and lies 4 bytes off a 16-byte boundary (scalar row stores), and the reference's contract (the kernel adds
    onto what the caller put there; model/norm_dist.py:37 zero-fills, here a constant, which must come back added).
    Run twice: the sums are rounded once from double bins, so the bits must not depend on the scheduling."""
    from gpu_common import DEV, cpp, say
    B, CO, CI, G, HW = shape
    say("inf_backward weight alone", shape, "accumulate" if accumulate else "overwrite, misaligned")
    x, w = make_inputs(B, CO, CI, G, HW, seed=sum(shape) + 1, quantize=8)
    _, ep = oracle.inf_dist_forward(x, w, G)
    go = torch.randn(B, CO, HW, generator=gen(78))
    K = CI // G
    want = oracle.inf_dist_backward_weight(go, ep, CI, G)
    god, epd = go.to(DEV), ep.to(DEV)
    got = []
    for _ in range(2):
        if accumulate:
            gw = torch.full((CO, K), 0.5, device=DEV)
            cpp.inf_dist_backward_weight(god, epd, gw, G)
            torch.cuda.synchronize()
            got.append(gw.cpu())
        else:
            flat = torch.full((CO * K + 1,), float("nan"), device=DEV)
            gw = flat[1:].view(CO, K)
            assert gw.data_ptr() % 16 == 4
            cpp.inf_dist_backward_weight_overwrite(god, epd, gw, G)
            torch.cuda.synchronize()
            assert bool(torch.isnan(flat[0]))              # the element in front of the view is not touched
            got.append(gw.cpu())
    assert torch.equal(got[0], got[1])
    if accumulate:
        # exact where nothing was added; elsewhere the float nearest to 0.5 + sum
        assert bool((got[0][want == 0] == 0.5).all())
        assert_scatter_close(got[0], (want.double() + 0.5))
    else:
        assert_scatter_close(got[0], want)
        assert not bool((got[0] == 0).logical_and(torch.signbit(got[0])).any())   # no -0.0 where nothing landed


def test_conv_layer_without_a_gradient_takes_the_values_only_forward():
    """NormDistConv at p = inf in evaluation under torch.no_grad(): the same output as with gradients enabled
    (which records the argmax), from the kernel without pos."""
    from gpu_common import DEV, pkg
    torch.manual_seed(3)
    layer = pkg.NormDistConv(32, 64, 3, stride=1, padding=1, group=2, p=float("inf"), bias=True, mean_normalize=True).to(DEV).eval()
    x = torch.rand(4, 32, 32, 32, device=DEV)
    y1 = layer(x)[0]
    with torch.no_grad():
        y0 = layer(x)[0]
    assert y1.requires_grad and not y0.requires_grad and torch.equal(y0, y1.detach())


@pytest.mark.parametrize("K", [2_000_000, 2_100_000, 2_100_002])
def test_forward_kernels_with_very_long_rows(K):
    """The fc panels are read through 32-bit buffer offsets, which cover tile rows of up to 2 GB: 258 rows of
    K = 2 000 000 floats still fit, K = 2 100 000 does not and takes the path with 64-bit addresses (as does a K
    that is not a multiple of four).  All three forward kernels, values and indices against the oracle."""
    from gpu_common import DEV, cpp, gpu_inf_forward, say
    say("long rows", K)
    g = torch.Generator().manual_seed(K % 1000)
    x = torch.rand(3, K, 1, generator=g)
    w = torch.rand(5, K, generator=g)
    out, pos = gpu_inf_forward(x, w, 1)
    eo, ep = oracle.inf_dist_forward(x, w, 1)
    assert torch.equal(out, eo) and torch.equal(pos, ep)
    lo, up = x - 0.01, x + 0.02
    L = torch.empty(3, 5, 1, device=DEV)
    U = torch.empty(3, 5, 1, device=DEV)
    cpp.inf_dist_bound_forward(lo.to(DEV), up.to(DEV), w.to(DEV), L, U, 1)
    eL, eU = oracle.inf_dist_bound_forward(lo, up, w, 1)
    assert torch.equal(L.cpu(), eL) and torch.equal(U.cpu(), eU)
    o8 = torch.empty(3, 5, 1, device=DEV)
    cpp.norm_dist_forward(x.to(DEV), w.to(DEV), o8, 1, 8.0)
    e8 = oracle.norm_dist_forward(x, w, 1, 8.0)
    assert torch.allclose(o8.cpu(), e8.float(), rtol=1e-4, atol=ATOL)   # a float32 sum of two million terms


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("B,NG,G", [(1024, 160, 1), (1100, 400, 2), (1536, 96, 1), (2048, 80, 2)])
def test_forward_kernels_with_many_row_tiles(B, NG, G, tile):
    """More row tiles than the workgroups that share an L2 cover per column tile: the launchers walk the row tiles
    in blocks then.  Every tile of the output must still be computed exactly once: the L_inf forward (values and
    indices), its values-only form and the interval kernel against the oracle, on every tiling."""
    from gpu_common import DEV, cpp, gpu_inf_forward, say, set_tile
    say("many row tiles", B, NG, G, tile)
    K = 48
    g = torch.Generator().manual_seed(B + NG + G)
    x = torch.rand(B, G * K, 1, generator=g)
    w = torch.randn(G * NG, K, generator=g)
    eo, ep = oracle.inf_dist_forward(x, w, G)
    set_tile(tile)
    try:
        out, pos = gpu_inf_forward(x, w, G)
        assert torch.equal(out, eo) and torch.equal(pos, ep)
        v = torch.full((B, G * NG, 1), -1.0, device=DEV)
        if cpp.inf_dist_forward_values(x.to(DEV), w.to(DEV), v, G):
            assert torch.equal(v.cpu(), eo)
        lo, up = x - 0.01, x + 0.02
        L = torch.empty(B, G * NG, 1, device=DEV)
        U = torch.empty(B, G * NG, 1, device=DEV)
        cpp.inf_dist_bound_forward(lo.to(DEV), up.to(DEV), w.to(DEV), L, U, G)
        eL, eU = oracle.inf_dist_bound_forward(lo, up, w, G)
        assert torch.equal(L.cpu(), eL) and torch.equal(U.cpu(), eU)
    finally:
        set_tile(-1)


# B, CO, CI, G, HW -- unfolded-conv layouts for the kernel that keeps a tile's whole reduction axis in LDS
SHORTK_SHAPES = [
    (2, 64, 64, 2, 64),       # K = 32: one window per k range
    (4, 128, 1152, 4, 100),   # the 3x3 conv layer over 32 channels per group (K = 288); rows end inside a tile
    (3, 40, 27, 1, 36),       # K = 27 (three channels): padded k, outputs end inside a tile (40 = 32 + 8)
    (2, 20, 100, 1, 16),      # K not a multiple of 8, one output tile with a tail, a single partial row tile
    (1, 70, 200, 2, 1024),    # 35 outputs per group, a whole 32 x 32 image
    (5, 33, 9, 1, 4),         # tiny: one group of four rows per image
    (2, 32, 320, 1, 32),      # K = 320: the longest reduction the kernel takes
    (70, 64, 96, 2, 64),      # more tiles than CUs: 140 row tiles x 2 groups, runs of tiles that change group
]


@pytest.mark.parametrize("quant", [None, 8])
@pytest.mark.parametrize("shape", SHORTK_SHAPES)
def test_inf_forward_short_reduction_kernel_bit_exact(shape, quant):
    """Values and indices of the LDS-resident short-K kernel (the default for these shapes) against the oracle, with
    quantised inputs for ties inside and across windows and k ranges; the same shapes through the tiled kernel
    (override 1) must agree as well."""
    from gpu_common import gpu_inf_forward, say, set_tile
    B, CO, CI, G, HW = shape
    say("inf_forward short-K", shape, "quant", quant)
    x, w = make_inputs(B, CO, CI, G, HW, seed=7 + sum(shape), quantize=quant)
    eo, ep = oracle.inf_dist_forward(x, w, G)
    set_tile(-1)
    out, pos = gpu_inf_forward(x, w, G)
    assert torch.equal(out, eo)
    assert torch.equal(pos, ep)
    set_tile(1)
    out, pos = gpu_inf_forward(x, w, G)
    assert torch.equal(out, eo) and torch.equal(pos, ep)


def test_inf_forward_short_reduction_kernel_specials():
    """NaN never wins, infinities do, an all-equal row gives (0, 0), and the sign bit follows x - w < 0, in the
    conv layout through the short-K kernel (reference model/inf_dist_cuda.cu:36-43)."""
    from gpu_common import gpu_inf_forward, set_tile
    nan, inf = float("nan"), float("inf")
    g = gen(77)
    x = torch.rand(2, 24, 8, generator=g)
    w = torch.randn(20, 24, generator=g) * 0.2
    x[0, 3, 1] = nan
    x[0, :, 2] = nan
    x[1, 5, 0] = inf
    x[1, 7, 4] = -inf
    x[1, 9, 4] = inf          # two infinite differences in one row: the lower k wins
    x[0, :, 5] = 0.25
    w[2, :] = 0.25            # row 5 of image 0 equals weight row 2 everywhere: value 0, pos 0
    x[1, :, 6] = 0.0
    w[4, :] = 0.0
    w[4, 11] = 0.5            # only k = 11 differs, x - w < 0
    set_tile(-1)
    out, pos = gpu_inf_forward(x, w, 1)
    eo, ep = oracle.inf_dist_forward(x, w, 1, literal=True)
    assert torch.equal(out, eo) and torch.equal(pos, ep)
    assert out[0, 2, 5].item() == 0.0 and pos[0, 2, 5].item() == 0
    assert pos[1, 4, 6].item() == (11 | SIGN)
    assert pos[1, 0, 4].item() == (7 | SIGN) and out[1, 0, 4].item() == inf


def test_inf_forward_known_answers_and_specials():
    from gpu_common import gpu_inf_forward
    nan, inf = float("nan"), float("inf")
    x = torch.tensor([[0.0, 2.0, 0.0], [2.0, 0.0, 0.0], [1.0, 1.0, 1.0], [nan, 1.0, 0.5], [nan, nan, nan],
                      [0.0, inf, 2.0], [0.0, -inf, inf]]).reshape(7, 3, 1)
    w = torch.tensor([[1.0, 1.0, 1.0], [0.0, 0.0, 0.0]])
    out, pos = gpu_inf_forward(x, w, 1)
    eo, ep = oracle.inf_dist_forward(x, w, 1, literal=True)
    assert torch.equal(out, eo) and torch.equal(pos, ep)
    assert pos[0, 0, 0].item() == (0 | SIGN) and pos[1, 0, 0].item() == 0 and pos[2, 0, 0].item() == 0


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("shape", SHAPES)
def test_bound_forward_bit_exact(shape, tile):
    from gpu_common import gpu_bound_forward, say, set_tile
    B, CO, CI, G, HW = shape
    say("bound_forward", shape, "tile", tile)
    x, w = make_inputs(B, CO, CI, G, HW, seed=1 + sum(shape))
    lo, up = (x - 8 / 255).clamp(0, 1).contiguous(), (x + 8 / 255).clamp(0, 1).contiguous()
    set_tile(tile)
    ol, ou = gpu_bound_forward(lo, up, w, G)
    el, eu = oracle.inf_dist_bound_forward(lo, up, w, G)
    assert torch.equal(ol, el) and torch.equal(ou, eu)
    # degenerate box reproduces the value forward bit for bit
    ol, ou = gpu_bound_forward(x, x, w, G)
    ev, _ = oracle.inf_dist_forward(x, w, G)
    assert torch.equal(ol, ev) and torch.equal(ou, ev)


@pytest.mark.parametrize("shape", [(33, 100, 77, 1, 1), (130, 70, 260, 1, 1), (2, 64, 64, 2, 64)])
def test_bound_forward_irregular_boxes_match_reference_predicate(shape):
    # lower > upper, NaN and infinities: the kernel must fall back to the literal predicate
    from gpu_common import gpu_bound_forward
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=9)
    g = gen(4)
    lo = (x - 0.1).contiguous()
    up = (x + 0.1).contiguous()
    flip = torch.rand(x.shape, generator=g) < 0.05
    lo2 = torch.where(flip, up, lo).contiguous()
    up2 = torch.where(flip, lo, up).contiguous()
    lo2[0, 0, 0] = float("nan")
    up2[-1, -1, -1] = float("inf")
    w2 = w.clone()
    w2[0, 0] = float("-inf")
    for (a, b, ww) in ((lo2, up2, w), (lo, up, w2)):
        ol, ou = gpu_bound_forward(a, b, ww, G)
        el, eu = oracle.inf_dist_bound_forward(a, b, ww, G)
        assert torch.equal(torch.nan_to_num(ol, nan=-1.0), torch.nan_to_num(el, nan=-1.0))
        assert torch.equal(torch.nan_to_num(ou, nan=-1.0), torch.nan_to_num(eu, nan=-1.0))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("overwrite", [False, True])
def test_inf_backward(shape, overwrite):
    from gpu_common import DEV, cpp, say
    B, CO, CI, G, HW = shape
    say("inf_backward", shape, "overwrite", overwrite)
    x, w = make_inputs(B, CO, CI, G, HW, seed=2 + sum(shape), quantize=16)
    _, pos = oracle.inf_dist_forward(x, w, G)
    go = torch.randn(B, CO, HW, generator=gen(5))
    ex = oracle.inf_dist_backward_input(go, pos, CI, G)
    ew = oracle.inf_dist_backward_weight(go, pos, CI, G)
    if overwrite:
        gx = torch.full((B, CI, HW), float("nan"), device=DEV)
        gw = torch.full((CO, CI // G), float("nan"), device=DEV)
        cpp.inf_dist_backward_input_overwrite(go.to(DEV), pos.to(DEV), gx, G)
        cpp.inf_dist_backward_weight_overwrite(go.to(DEV), pos.to(DEV), gw, G)
    else:
        gx = torch.full((B, CI, HW), 0.5, device=DEV)
        gw = torch.full((CO, CI // G), -0.25, device=DEV)
        cpp.inf_dist_backward_input(go.to(DEV), pos.to(DEV), gx, G)
        cpp.inf_dist_backward_weight(go.to(DEV), pos.to(DEV), gw, G)
        ex, ew = ex + 0.5, ew - 0.25
    torch.cuda.synchronize()
    torch.testing.assert_close(gx.cpu(), ex, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(gw.cpu(), ew, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("shape", SHAPES)
def test_value_bound_forward_bit_exact(shape, tile):
    """Values and both bounds from the one-pass kernel equal what the value kernel and the bound kernel give (the
    oracle's), bit for bit; with a mean and a bias every channel leaves as (v - mean) + bias in float32."""
    from gpu_common import gpu_value_bound_forward, say, set_tile
    B, CO, CI, G, HW = shape
    say("value_bound_forward", shape, "tile", tile)
    x, w = make_inputs(B, CO, CI, G, HW, seed=1 + sum(shape), quantize=8 if tile == 1 else None)
    lo, up = (x - 8 / 255).clamp(0, 1).contiguous(), (x + 8 / 255).clamp(0, 1).contiguous()
    ev, _ = oracle.inf_dist_forward(x, w, G)
    el, eu = oracle.inf_dist_bound_forward(lo, up, w, G)
    set_tile(tile)
    ov, ol, ou = gpu_value_bound_forward(x, lo, up, w, G)
    assert torch.equal(ov, ev) and torch.equal(ol, el) and torch.equal(ou, eu)
    mean, bias = torch.randn(CO, generator=gen(61)), torch.randn(CO, generator=gen(62))
    for m_, b_ in ((mean, None), (None, bias), (mean, bias)):
        ov, ol, ou = gpu_value_bound_forward(x, lo, up, w, G, m_, b_)
        for got, want in ((ov, ev), (ol, el), (ou, eu)):
            if m_ is not None:
                want = want - m_.view(1, CO, 1)
            if b_ is not None:
                want = want + b_.view(1, CO, 1)
            assert torch.equal(got, want)


@pytest.mark.parametrize("shape", [(33, 100, 77, 1, 1), (130, 70, 260, 1, 1), (2, 64, 64, 2, 64), (40, 10, 300, 1, 1)])
def test_value_bound_forward_irregular_boxes(shape):
    """lower > upper, NaN and infinities in the box, the point or the weights: the reference's literal predicate."""
    from gpu_common import gpu_value_bound_forward
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=9)
    g = gen(4)
    lo, up = (x - 0.1).contiguous(), (x + 0.1).contiguous()
    flip = torch.rand(x.shape, generator=g) < 0.05
    lo2, up2 = torch.where(flip, up, lo).contiguous(), torch.where(flip, lo, up).contiguous()
    lo2[0, 0, 0] = float("nan")
    up2[-1, -1, -1] = float("inf")
    x2 = x.clone()
    x2[0, 1, 0], x2[-1, 0, -1] = float("nan"), float("-inf")
    w2 = w.clone()
    w2[0, 0] = float("-inf")
    same = lambda a, b: torch.equal(torch.nan_to_num(a, nan=-1.0), torch.nan_to_num(b, nan=-1.0))
    for (xx, a, b, ww) in ((x2, lo2, up2, w), (x, lo, up, w2)):
        ov, ol, ou = gpu_value_bound_forward(xx, a, b, ww, G)
        ev, _ = oracle.inf_dist_forward(xx, ww, G, literal=True)
        el, eu = oracle.inf_dist_bound_forward(a, b, ww, G)
        assert same(ov, ev) and same(ol, el) and same(ou, eu)


def test_layers_with_few_outputs_certify_through_the_one_pass_kernel():
    """In evaluation mode without gradients, a layer without a window and with at most 16 outputs per group takes
    values and bounds from the one-pass kernel, running mean and bias included: same numbers as the separate
    kernels, bit for bit."""
    from gpu_common import DEV, pkg
    torch.manual_seed(3)
    for bias, mean_normalize, group, hw in ((True, True, 1, 1), (False, True, 2, 1), (True, False, 1, 3), (False, False, 4, 2)):
        co = 10 * group
        layer = pkg.NormDistConv(120, co, 1, group=group, p=float("inf"), bias=bias, mean_normalize=mean_normalize).to(DEV)
        with torch.no_grad():
            layer.weight.copy_(torch.randn(co, 120 // group, 1, 1))
            if bias:
                layer.bias.copy_(torch.randn(co))
            if mean_normalize:
                layer.normalize.running_mean.copy_(torch.randn(co))
        layer.eval()
        x = torch.rand(37, 120, hw, hw, generator=gen(71)).to(DEV)
        lo, up = x - 0.02, x + 0.02
        with torch.no_grad():
            assert layer._value_and_bounds_in_one_pass(x, lo, up)
            fused = layer(x, lo, up)
            layer.FUSED_VALUE_BOUND_MAX_OUTPUTS = 0
            assert not layer._value_and_bounds_in_one_pass(x, lo, up)
            separate = layer(x, lo, up)
        assert all(torch.equal(a, b) for a, b in zip(fused, separate))
        del layer.FUSED_VALUE_BOUND_MAX_OUTPUTS
        y, l, u = layer(x.requires_grad_(True), lo, up)      # with gradients enabled: the separate kernels, with autograd
        assert y.requires_grad and torch.equal(y.detach(), fused[0]) and torch.equal(l, fused[1])


PNORM_SHAPES = [s for s in SHAPES if s[1] * s[2] * s[0] * s[4] <= 40_000_000]


@pytest.mark.parametrize("tile", [-1, 0, 2])
@pytest.mark.parametrize("shape", PNORM_SHAPES)
@pytest.mark.parametrize("p", [8.0, 2.0, 3.5, 37.0, 1000.0])
def test_norm_forward(shape, tile, p):
    from gpu_common import gpu_norm_forward, say, set_tile
    B, CO, CI, G, HW = shape
    say("norm_forward", shape, "tile", tile, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=3 + sum(shape))
    set_tile(tile)
    out = gpu_norm_forward(x, w, G, p)
    torch.testing.assert_close(out, oracle.norm_dist_forward(x, w, G, p), rtol=RTOL, atol=ATOL)


def test_norm_forward_scale_robust_and_seeded():
    from gpu_common import gpu_norm_forward
    x, w = make_inputs(40, 50, 132, 1, 1, seed=4)
    for scale in (1e-6, 1.0, 1e6, 1e18):
        xs, ws = (x * scale).contiguous(), (w * scale).contiguous()
        out = gpu_norm_forward(xs, ws, 1, 8.0)
        torch.testing.assert_close(out, oracle.norm_dist_forward(xs, ws, 1, 8.0), rtol=RTOL, atol=0)
    same = torch.full((3, 8, 1), 0.25)
    out = gpu_norm_forward(same, torch.full((17, 8), 0.25), 1, 8.0)
    torch.testing.assert_close(out, oracle.norm_dist_forward(same, torch.full((17, 8), 0.25), 1, 8.0), rtol=1e-4,
                               atol=0)


@pytest.mark.parametrize("tile", [-1, 0, 1])
@pytest.mark.parametrize("p", [2.0, 3.0, 8.0, 3.5, 16.5, 37.0, 64.0, 64.5])
@pytest.mark.parametrize("profile", ["growing", "shrinking", "spike", "tiny"])
def test_norm_forward_magnitude_jumps_between_chunks(profile, p, tile):
    """|x - w| changes by orders of magnitude from one 32-wide chunk of k to the next: the kernel
    that sweeps a chunk once with the scale of earlier chunks has to notice the overflow and go
    back over the chunk (growing, spike), and must not lose small later terms (shrinking)."""
    from gpu_common import gpu_norm_forward, say, set_tile
    B, CO, K = 70, 90, 416
    say("norm_forward magnitude jumps", profile, "p", p, "tile", tile)
    x, w = make_inputs(B, CO, K, 1, 1, seed=11)
    chunk = torch.arange(K) // 32
    if profile == "growing":
        mag = 10.0 ** (2.0 * chunk.float() - 6.0)            # 1e-6 ... 1e18
    elif profile == "shrinking":
        mag = 10.0 ** (6.0 - 1.0 * chunk.float())
    elif profile == "spike":
        mag = torch.ones(K)
        mag[200:203] = 1e9
    else:
        mag = torch.full((K,), 1e-12)                         # the 1e-10 seeds of the reference matter here
    xs = (x * mag.view(1, K, 1)).contiguous()
    ws = (w * mag.view(1, K)).contiguous()
    set_tile(tile)
    out = gpu_norm_forward(xs, ws, 1, p)
    set_tile(-1)
    torch.testing.assert_close(out, oracle.norm_dist_forward(xs, ws, 1, p), rtol=RTOL, atol=0)


@pytest.mark.parametrize("shape", PNORM_SHAPES)
@pytest.mark.parametrize("p", [8.0, 2.0, 3.0, 4.0, 5.5, 100.0])
def test_norm_backward(shape, p):
    from gpu_common import DEV, cpp, say
    B, CO, CI, G, HW = shape
    say("norm_backward", shape, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=6 + sum(shape))
    go = torch.randn(B, CO, HW, generator=gen(7))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.full((CO, CI // G), 0.125, device=DEV)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV))
    cpp.norm_dist_backward_input(*args, gx, G, p)
    cpp.norm_dist_backward_weight(*args, gw, G, p)
    torch.cuda.synchronize()
    # rel 1e-5 / abs 1e-6, the absolute part relative to the magnitude of the summed terms
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu() - 0.125, ew, mw, p, RTOL, ATOL)


# B, CO, CI, G, HW -- shapes the register-tiled grad_input kernel can take (K % 4 == 0; NG % 4 == 0 or HW % 4 == 0)
TILED_BACKWARD_SHAPES = [
    (130, 72, 260, 1, 1),     # fc: row tail, column tails of the 80- and 64-wide tiles, reduction shorter than two stages
    (64, 96, 96, 3, 1),       # groups, one stage of exactly 32 outputs per group
    (200, 300, 164, 1, 1),    # several stages with a ragged last one (300 = 4 * 64 + 44), K = 164: a tile's last group of four
    (2, 64, 64, 2, 64),       # conv layout
    (3, 40, 36, 1, 100),      # conv layout: rows end inside a tile (300 rows), images change inside a tile
    (4, 128, 1152, 4, 100),   # the grouped 3x3 conv layer shape at a small image
]


@pytest.mark.parametrize("tile", [0, 1])
@pytest.mark.parametrize("p", [8.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("shape", TILED_BACKWARD_SHAPES)
def test_norm_backward_input_register_tiled(shape, p, tile):
    """grad_input of the multiply-only exponents on the register-tiled kernel (forced with the tile override:
    0 = 128 x 80 tiles, 1 = 128 x 64; by itself it only takes large layers) against the oracle, and against the
    64 x 64 kernel it replaces there (override 2), with the same tolerance."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = shape
    say("norm_backward_input tiled", shape, "p", p, "tile", tile)
    x, w = make_inputs(B, CO, CI, G, HW, seed=16 + sum(shape))
    go = torch.randn(B, CO, HW, generator=gen(17))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV))
    for choice in (tile, 2):
        set_tile(choice)
        gx = torch.full((B, CI, HW), float("nan"), device=DEV)
        cpp.norm_dist_backward_input(*args, gx, G, p)
        torch.cuda.synchronize()
        assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)


@pytest.mark.parametrize("tile", [0, 1])
@pytest.mark.parametrize("p", [8.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("shape", [sh for sh in TILED_BACKWARD_SHAPES if sh[4] == 1] + [(515, 140, 100, 1, 1), (70, 200, 132, 1, 1)])
def test_norm_backward_weight_register_tiled(shape, p, tile):
    """grad_weight of the multiply-only exponents in the fc layout on the register-tiled kernel (forced with the
    tile override) against the oracle; the kernel adds onto the buffer it is given (reference contract)."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = shape
    say("norm_backward_weight tiled", shape, "p", p, "tile", tile)
    x, w = make_inputs(B, CO, CI, G, HW, seed=26 + sum(shape))
    go = torch.randn(B, CO, HW, generator=gen(27))
    out = oracle.norm_dist_forward(x, w, G, p)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV))
    for choice in (tile, 2):
        set_tile(choice)
        gw = torch.full((CO, CI // G), 0.125, device=DEV)
        cpp.norm_dist_backward_weight(*args, gw, G, p)
        torch.cuda.synchronize()
        assert_sum_close(gw.cpu() - 0.125, ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [2.0, 4.0, 8.0])
@pytest.mark.parametrize("scale", [1e-6, 1.0, 1e6, "mixed"])
def test_norm_backward_weight_register_tiled_at_every_scale(scale, p):
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = 200, 72, 132, 1, 1
    say("norm_backward_weight tiled scale", scale, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=43)
    if scale == "mixed":
        x = x * torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0])[torch.arange(B) % 5].view(B, 1, 1)
    else:
        x, w = x * scale, w * scale
    x, w = x.contiguous(), w.contiguous()
    go = torch.randn(B, CO, HW, generator=gen(28))
    out = oracle.norm_dist_forward(x, w, G, p)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    set_tile(0)
    gw = torch.zeros((CO, CI // G), device=DEV)
    cpp.norm_dist_backward_weight(go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV), gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [2.0, 3.0, 4.0, 8.0])
@pytest.mark.parametrize("scale", [1e-6, 3e-4, 1.0, 5e3, 1e6, "mixed", "one tiny row"])
def test_norm_backward_input_register_tiled_at_every_scale(scale, p):
    """The tiled kernel takes powers of raw differences only while every output of a stage lies within [2^-12, 2^12];
    a stage that holds one outside goes the normalised way.  Tiny and huge data, rows of very different magnitude
    in one stage, and a single tiny row among ordinary ones (so that some stages switch and others do not)."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = 70, 200, 132, 1, 1
    say("norm_backward_input tiled scale", scale, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=33)
    if scale == "mixed":
        x = x * torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0])[torch.arange(B) % 5].view(B, 1, 1)
    elif scale == "one tiny row":
        x[17] *= 1e-7
        w[100:] *= 1e-7          # only the outputs of the later stages are tiny for that row
    else:
        x, w = x * scale, w * scale
    x, w = x.contiguous(), w.contiguous()
    go = torch.randn(B, CO, HW, generator=gen(18))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    set_tile(0)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    cpp.norm_dist_backward_input(go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV), gx, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [2.0, 3.0, 4.0, 8.0])
@pytest.mark.parametrize("scale", [1e-9, 1e-6, 2e-4, 3e-4, 1.0, 3e3, 5e3, 1e6, 1e15, "mixed"])
def test_norm_forward_at_every_scale(scale, p):
    """Small integer p sums raw powers while the running scales of a wave lie within 2^(+-96/p) and takes the
    normalised path outside (and for the first chunk, and on overflow): every scale, the switch-over points and
    rows of very different magnitude must give the same relative accuracy."""
    from gpu_common import gpu_norm_forward, say
    say("norm_forward scale", scale, "p", p)
    x, w = make_inputs(70, 96, 260, 1, 1, seed=29)
    if scale == "mixed":
        rows = torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0])[torch.arange(70) % 5].view(70, 1, 1)
        x = x * rows
    else:
        x, w = x * scale, w * scale
    out = gpu_norm_forward(x.contiguous(), w.contiguous(), 1, p)
    torch.testing.assert_close(out, oracle.norm_dist_forward(x.contiguous(), w.contiguous(), 1, p), rtol=RTOL, atol=0)


@pytest.mark.parametrize("p", [2.0, 3.0, 4.0, 8.0])
@pytest.mark.parametrize("scale", [1e-6, 3e-4, 1.0, 5e3, 1e6, "mixed"])
def test_norm_backward_at_every_scale(scale, p):
    """The small integer exponents factor the term as (c * rinv^(p-1)) * (x-w)^(p-1) only while every output of a
    stage lies within [2^-12, 2^12]; outside (tiny or huge data, or rows of very different magnitude in one stage)
    the normalised form is used.  Both must meet the tolerance, relative to the magnitude of the summed terms."""
    from gpu_common import DEV, cpp, say
    B, CO, CI, G, HW = 70, 96, 130, 1, 1
    say("norm_backward scale", scale, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=23)
    if scale == "mixed":
        rows = torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0])[torch.arange(B) % 5].view(B, 1, 1)
        x, w = x * rows, w * 1.0          # some rows tiny, some huge, weights of order one
    else:
        x, w = x * scale, w * scale
    go = torch.randn(B, CO, HW, generator=gen(8))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.zeros((CO, CI // G), device=DEV)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV))
    cpp.norm_dist_backward_input(*args, gx, G, p)
    cpp.norm_dist_backward_weight(*args, gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [64.0, 100.5, 128.0, 300.0, 1000.0])
@pytest.mark.parametrize("data", ["normal", "flat", "ties", "tiny", "mixed", "conv", "grouped"])
def test_norm_large_exponents(data, p):
    """From p = 64 (backward) and p = 128 (forward) the kernels test whether a row of terms can matter before they
    take its powers, and pass over rows of negligible terms.  Normal weights: nearly every row is passed over.
    Flat: differences crowd below the maximum, most rows count (the forward gives up testing).  Ties: many terms
    equal the maximum exactly.  Tiny: everything below the reference's 1e-10 seed, where nothing is negligible.
    Mixed: rows of very different magnitude.  All must meet the same tolerance as every other exponent."""
    from gpu_common import DEV, cpp, gpu_norm_forward, say
    say("norm large exponent", data, "p", p)
    B, CO, CI, G, HW = 70, 96, 2200, 1, 1      # the tests run from 1024 (backward) and 2048 (forward) inputs per output
    if data == "conv":
        B, CO, CI, G, HW = 3, 40, 2100, 1, 50
    elif data == "grouped":
        B, CO, CI, G, HW = 40, 48, 4200, 2, 1
    g = gen(31)
    x = torch.randn(B, CI, HW, generator=g)
    w = torch.randn(CO, CI // G, generator=g)
    if data == "flat":
        x, w = torch.rand(B, CI, HW, generator=g), w * 0.01
    elif data == "ties":
        x, w = torch.randint(0, 2, (B, CI, HW), generator=g).float(), torch.zeros(CO, CI // G)
    elif data == "tiny":
        x, w = x * 1e-12, w * 1e-12
    elif data == "mixed":
        x = x * torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0])[torch.arange(B) % 5].view(B, 1, 1)
    x, w = x.contiguous(), w.contiguous()
    want = oracle.norm_dist_forward(x, w, G, p)
    out = gpu_norm_forward(x, w, G, p)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=0)
    go = torch.randn(B, CO, HW, generator=gen(9))
    ex, mx = oracle.norm_dist_backward_input(go, x, w, want, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, want, G, p, with_abs_terms=True)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.zeros((CO, CI // G), device=DEV)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), want.to(DEV))
    cpp.norm_dist_backward_input(*args, gx, G, p)
    cpp.norm_dist_backward_weight(*args, gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)
    # the call for both gradients, on the kernels that evaluate every term once (forced on), which pass over the
    # same negligible rows for both sums
    from gpu_common import set_tile
    set_tile(0)
    gx2 = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw2 = torch.zeros((CO, CI // G), device=DEV)
    cpp.norm_dist_backward(*args, gx2, gw2, G, p)
    torch.cuda.synchronize()
    set_tile(-1)
    assert_sum_close(gx2.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw2.cpu(), ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("shape", [(512, 5120, 1), (37, 10, 1), (1030, 50, 1), (600, 36, 1), (6, 5, 12), (4, 3, 7),
                                   (16, 8, 1024)])
def test_mean_shift_kernel(shape):
    """One-kernel per-channel mean shift (training-mode MeanNorm, reference model/norm_dist.py:85-96)
    against the closed form in float64; also the mean it reports and the running mean it moves."""
    from gpu_common import DEV, cpp, say
    say("mean_shift", shape)
    B, C, L = shape
    x = torch.randn(B, C, L, generator=gen(21)) + torch.linspace(-3, 3, C).view(1, C, 1)
    running = torch.linspace(-1, 1, C)
    mean64 = x.double().mean(dim=(0, 2))
    xd = x.to(DEV)
    y = torch.full_like(xd, float("nan"))
    mean_out = torch.empty(C, device=DEV)
    rm = running.to(DEV)
    cpp.mean_shift(xd, y, mean_out, rm, 0.1)
    torch.cuda.synchronize()
    torch.testing.assert_close(mean_out.cpu().double(), mean64, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(y.cpu().double(), x.double() - mean64.view(1, C, 1), rtol=1e-6, atol=2e-6)
    torch.testing.assert_close(rm.cpu().double(), 0.9 * running.double() + 0.1 * mean64, rtol=1e-6, atol=1e-6)
    y2 = torch.empty_like(xd)                      # the optional outputs left out
    cpp.mean_shift(xd, y2)
    torch.cuda.synchronize()
    assert torch.equal(y2, y)


def test_mean_norm_module_on_gpu_matches_cpu_module():
    from gpu_common import DEV, pkg
    for shape in ((64, 12), (8, 6, 5, 5)):
        x = torch.randn(*shape, generator=gen(22))
        up = torch.randn(*shape, generator=gen(23))
        ref, dev = pkg.MeanNorm(shape[1]).train(), pkg.MeanNorm(shape[1]).train().to(DEV)
        xa, xb = x.clone().requires_grad_(True), x.to(DEV).requires_grad_(True)
        ref(xa).backward(up)
        out = dev(xb)
        out.backward(up.to(DEV))
        torch.cuda.synchronize()
        torch.testing.assert_close(out.detach().cpu(), ref(x).detach(), rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=1e-6, atol=1e-6)
        # two training-mode calls on the CPU module, one on the GPU module
        torch.testing.assert_close(dev.running_mean.cpu(), 0.1 * x.mean(dim=tuple(d for d in range(x.dim()) if d != 1)),
                                   rtol=1e-5, atol=1e-6)
        dev.eval()
        torch.testing.assert_close(dev(x.to(DEV)).cpu(), x - dev.running_mean.cpu().view(1, -1, *([1] * (x.dim() - 2))),
                                   rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(64, 5120), (37, 50), (128, 288), (10, 5120), (33, 1), (5, 3, 3, 3), (300, 7)])
@pytest.mark.parametrize("p", [None, 2.0, 4.0, 8.0, 3.5, 37.0, 1000.0, float("inf")])
def test_adamw_lp_step_kernel(shape, p):
    """The fused optimizer step (reference adamw.py:36-85) against the double-precision oracle over
    three steps; moments and parameter within float32 rounding."""
    from gpu_common import DEV, cpp, say
    say("adamw_lp_step", shape, "p", p)
    g = gen(41)
    w = torch.randn(*shape, generator=g) * 0.5
    if len(shape) == 2 and shape[1] >= 50:
        w[1, 7], w[1, 30] = 3.0, -3.0                     # a tie for the largest entry: the first decays at p = inf
    m, v = torch.zeros_like(w), torch.zeros_like(w)
    wd_, md, vd = w.to(DEV), m.to(DEV), v.to(DEV)
    hp = dict(lr=0.03, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.25)
    for step in (1, 2, 3):
        grad = torch.randn(*shape, generator=g)
        rows = w.view(w.size(0), -1)
        oracle.adamw_lp_step(rows, grad.view_as(rows), m.view_as(rows), v.view_as(rows), p, hp["lr"], hp["betas"],
                             hp["eps"], hp["weight_decay"], step)
        cpp.adamw_lp_step(wd_, grad.to(DEV), md, vd, p, hp["lr"], hp["betas"][0], hp["betas"][1], hp["eps"],
                          hp["weight_decay"], step)
        torch.cuda.synchronize()
        torch.testing.assert_close(md.cpu(), m, rtol=1e-6, atol=2e-7)      # 0.9 m + 0.1 g can cancel
        torch.testing.assert_close(vd.cpu(), v, rtol=1e-6, atol=1e-9)
        torch.testing.assert_close(wd_.cpu(), w, rtol=1e-5, atol=1e-6)


def test_adamw_optimizer_on_gpu_follows_the_cpu_optimizer():
    from gpu_common import DEV, pkg
    for p in (8.0, float("inf")):
        torch.manual_seed(5)
        cpu_model = pkg.MLP(depth=3, width=1, input_dim=48, num_classes=10)
        gpu_model = pkg.MLP(depth=3, width=1, input_dim=48, num_classes=10)
        gpu_model.load_state_dict(cpu_model.state_dict())
        gpu_model = gpu_model.to(DEV)
        for mdl in (cpu_model, gpu_model):
            pkg.set_p_norm(mdl, p)
        oc, og = pkg.AdamW(cpu_model, lr=0.01, weight_decay=0.1), pkg.AdamW(gpu_model, lr=0.01, weight_decay=0.1)
        g = gen(43)
        for _ in range(3):
            for a, b in zip(cpu_model.parameters(), gpu_model.parameters()):
                a.grad = torch.randn(a.shape, generator=g)
                b.grad = a.grad.to(DEV)
            oc.step()
            og.step()
        torch.cuda.synchronize()
        for a, b in zip(cpu_model.parameters(), gpu_model.parameters()):
            torch.testing.assert_close(b.detach().cpu(), a.detach(), rtol=2e-5, atol=2e-6)


CONV_CASES = [  # B, C, H, W, k, stride, padding, dilation
    (2, 4, 8, 8, 3, 1, 1, 1), (3, 6, 9, 7, 3, 1, 0, 1), (2, 8, 12, 12, 3, 2, 1, 1), (1, 3, 11, 13, 5, 1, 2, 1),
    (2, 4, 10, 10, 3, 1, 2, 2), (4, 16, 32, 32, 3, 1, 1, 1), (2, 2, 6, 6, 2, 2, 0, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_unfold_and_fold_kernels(case):
    """Native patch extraction against torch.nn.functional.unfold (bit-equal: it only copies), and its
    adjoint against autograd through F.unfold."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, say
    say("unfold/fold", case)
    B, C, H, W, k, s_, p_, d_ = case
    img = torch.randn(B, C, H, W, generator=gen(51))
    ref = F.unfold(img, k, d_, p_, s_)
    cols = torch.full(ref.shape, float("nan"), device=DEV)
    cpp.unfold(img.to(DEV), cols, k, s_, p_, d_)
    torch.cuda.synchronize()
    assert torch.equal(cols.cpu(), ref)
    gcols = torch.randn(ref.shape, generator=gen(52))
    leaf = img.double().requires_grad_(True)
    F.unfold(leaf, k, d_, p_, s_).backward(gcols.double())
    gimg = torch.full(img.shape, float("nan"), device=DEV)
    cpp.fold(gcols.to(DEV), gimg, k, s_, p_, d_)
    torch.cuda.synchronize()
    torch.testing.assert_close(gimg.cpu().double(), leaf.grad, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("group", [1, 2])
@pytest.mark.parametrize("case", CONV_CASES)
def test_inf_backward_input_folded(case, group):
    """Scatter and fold fused, against the oracle's scatter into the columns followed by torch's fold."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, say
    B, C, H, W, k, s_, p_, d_ = case
    if C % group:
        pytest.skip("channels do not divide into the groups")
    say("inf_backward_input_folded", case, "group", group)
    CO = 6 * group
    img = torch.randn(B, C, H, W, generator=gen(53))
    w = torch.randn(CO, C // group * k * k, generator=gen(54)) * 0.5
    cols = F.unfold(img, k, d_, p_, s_).contiguous()
    _, pos = oracle.inf_dist_forward(cols, w, group)
    go = torch.randn(B, CO, cols.size(2), generator=gen(55))
    expect = F.fold(oracle.inf_dist_backward_input_f64(go, pos, cols.size(1), group), (H, W), k, d_, p_, s_)
    gimg = torch.full(img.shape, float("nan"), device=DEV)
    cpp.inf_dist_backward_input_folded(go.to(DEV), pos.to(DEV), gimg, group, k, s_, p_, d_)
    torch.cuda.synchronize()
    assert_scatter_close(gimg.cpu(), expect)


IMPLICIT_CASES = [  # B, C, H, W, CO, G, stride, padding
    (2, 4, 8, 8, 8, 1, 1, 1),        # one 8-wide segment per row
    (2, 8, 16, 16, 24, 2, 1, 1),     # groups, 12 outputs each
    (3, 6, 9, 16, 10, 1, 1, 1),      # odd height, channels padded up to the stage of four, ragged outputs
    (2, 3, 32, 32, 20, 1, 1, 1),     # first layer of the CIFAR net: 3 channels
    (2, 8, 16, 16, 16, 1, 2, 1),     # stride 2
    (2, 5, 17, 17, 12, 1, 2, 0),     # stride 2 without padding, odd image
    (1, 16, 32, 32, 96, 1, 1, 1),    # 96 outputs: two tiles of 48
    (2, 128, 32, 32, 128, 4, 1, 1),  # the benchmark layer at a small batch
    (2, 4, 10, 10, 8, 1, 1, 0),      # no padding
    (2, 4, 6, 6, 8, 1, 1, 2),        # padding wider than the window needs
    (1, 8, 8, 64, 40, 1, 1, 1),      # wide rows: eight segments
    (2, 72, 16, 16, 72, 1, 1, 1),    # many channels in one group
    (2, 16, 28, 28, 32, 1, 1, 1),    # MNIST-sized rows: 28 positions, the fourth segment half idle
    (2, 8, 13, 13, 16, 2, 1, 0),     # output width 11
    (2, 8, 21, 21, 12, 1, 2, 1),     # stride 2, output width 11
]


@pytest.mark.parametrize("rows", [0, 2])
@pytest.mark.parametrize("quant", [None, 8])
@pytest.mark.parametrize("case", IMPLICIT_CASES)
def test_inf_conv_forward_matches_column_path_bit_exact(case, quant, rows):
    """The kernel that reads the image directly against the oracle on torch's unfolded columns: values and
    first-argmax indices bit for bit (quantised inputs force ties, so the first index is what is checked)."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, pkg, say
    B, C, H, W, CO, G, s_, p_ = case
    say("inf_conv_forward", case, "quant", quant, "rows", rows)
    lib = pkg._lib.lib()
    assert lib.ldist_set_conv_rows_override(rows) == 0   # 0: the library's choice; 2: forced, small layers included
    if not cpp.inf_dist_conv_forward_supported(C, H, W, CO, G, 3, s_, p_, 1):
        assert rows == 0
        pytest.skip("left to the column path by the library")
    img = torch.randn(B, C, H, W, generator=gen(61))
    w = torch.randn(CO, C // G * 9, generator=gen(62)) * 0.7
    if quant:
        img, w = (img * quant).round() / quant, (w * quant).round() / quant
    cols = F.unfold(img, 3, 1, p_, s_).contiguous()
    eo, ep = oracle.inf_dist_forward(cols, w, G)
    out = torch.full(eo.shape, float("nan"), device=DEV)
    pos = torch.full(eo.shape, -7, device=DEV, dtype=torch.int32)
    cpp.inf_dist_conv_forward(img.to(DEV), w.to(DEV), out, pos, G, 3, s_, p_, 1)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), eo)
    assert torch.equal(pos.cpu(), ep)
    # the kernel without pos (for passes that no gradient follows): the same values
    only = torch.full(eo.shape, float("nan"), device=DEV)
    cpp.inf_dist_conv_forward_values(img.to(DEV), w.to(DEV), only, G, 3, s_, p_, 1)
    assert torch.equal(only.cpu(), eo)


STAGED_CASES = [  # B, C, H, W, CO, G, stride, padding: channels per group a multiple of four
    (2, 8, 16, 16, 24, 2, 1, 1), (2, 128, 32, 32, 128, 4, 1, 1), (2, 96, 32, 32, 96, 1, 1, 1),
    (2, 96, 32, 32, 192, 1, 2, 1), (1, 192, 16, 16, 192, 1, 1, 1), (2, 8, 17, 17, 12, 1, 2, 0),
    (1, 8, 8, 64, 40, 1, 1, 1), (2, 4, 6, 6, 8, 1, 1, 2), (3, 12, 9, 16, 10, 1, 1, 1),
    (2, 16, 28, 28, 32, 1, 1, 1), (2, 8, 21, 21, 12, 1, 2, 1),     # output widths 28 and 11: ragged last segment
]


@pytest.mark.parametrize("rows", [0, 3, 8])
@pytest.mark.parametrize("quant", [None, 8])
@pytest.mark.parametrize("case", STAGED_CASES)
def test_inf_conv_forward_staged_channels_bit_exact(case, quant, rows):
    """The variant that moves four channels at a time through LDS (many channels per group), forced for
    every case, against the oracle on torch's unfolded columns."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, pkg, say
    B, C, H, W, CO, G, s_, p_ = case
    say("inf_conv_forward staged", case, "quant", quant, "rows", rows)
    lib = pkg._lib.lib()
    assert lib.ldist_set_conv_staging_override(2) == 0 and lib.ldist_set_conv_rows_override(rows) == 0
    try:
        if not cpp.inf_dist_conv_forward_supported(C, H, W, CO, G, 3, s_, p_, 1):
            pytest.skip("left to the column path by the library")
        img = torch.randn(B, C, H, W, generator=gen(65))
        w = torch.randn(CO, C // G * 9, generator=gen(66)) * 0.7
        if quant:
            img, w = (img * quant).round() / quant, (w * quant).round() / quant
        eo, ep = oracle.inf_dist_forward(F.unfold(img, 3, 1, p_, s_).contiguous(), w, G)
        out = torch.full(eo.shape, float("nan"), device=DEV)
        pos = torch.full(eo.shape, -7, device=DEV, dtype=torch.int32)
        cpp.inf_dist_conv_forward(img.to(DEV), w.to(DEV), out, pos, G, 3, s_, p_, 1)
        only = torch.full(eo.shape, float("nan"), device=DEV)   # the same variant of the kernel without pos
        cpp.inf_dist_conv_forward_values(img.to(DEV), w.to(DEV), only, G, 3, s_, p_, 1)
        torch.cuda.synchronize()
    finally:
        lib.ldist_set_conv_staging_override(0)
    assert torch.equal(out.cpu(), eo)
    assert torch.equal(pos.cpu(), ep)
    assert torch.equal(only.cpu(), eo)


@pytest.mark.parametrize("rows", [1, 2, 3, 5, 8])
def test_inf_conv_forward_any_rows_per_workgroup(rows):
    """Forcing the number of output rows a workgroup owns (tails at the image bottom included) changes nothing."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, pkg, say
    say("inf_conv_forward rows", rows)
    B, C, H, W, CO, G = 2, 8, 12, 16, 16, 2
    img = torch.randn(B, C, H, W, generator=gen(63))
    img[0, 1, 3, 4] = float("nan")
    img[1, 2, 0, 0] = float("inf")
    w = torch.randn(CO, C // G * 9, generator=gen(64))
    eo, ep = oracle.inf_dist_forward(F.unfold(img, 3, 1, 1, 1).contiguous(), w, G, literal=True)
    out = torch.empty(eo.shape, device=DEV)
    pos = torch.empty(eo.shape, device=DEV, dtype=torch.int32)
    lib = pkg._lib.lib()
    assert lib.ldist_set_conv_rows_override(rows) == 0
    try:
        cpp.inf_dist_conv_forward(img.to(DEV), w.to(DEV), out, pos, G, 3, 1, 1, 1)
        torch.cuda.synchronize()
    finally:
        lib.ldist_set_conv_rows_override(0)
    assert torch.equal(out.cpu(), eo)
    assert torch.equal(pos.cpu(), ep)


def test_inf_conv_forward_refuses_what_it_does_not_cover():
    from gpu_common import DEV, cpp, pkg
    assert not cpp.inf_dist_conv_forward_supported(4, 16, 16, 8, 1, 5, 1, 2, 1)    # 5x5 window
    assert not cpp.inf_dist_conv_forward_supported(4, 16, 16, 8, 1, 3, 1, 2, 2)    # dilation
    img = torch.zeros(1, 4, 28, 28, device=DEV)
    w = torch.zeros(8, 100, device=DEV)
    out = torch.empty(1, 8, 784, device=DEV)
    pos = torch.empty(1, 8, 784, device=DEV, dtype=torch.int32)
    rc = pkg._lib.lib().ldist_inf_dist_conv_forward(img.data_ptr(), w.data_ptr(), 1, 4, 28, 28, 8, 1, 5, 5, 1, 2, 1,
                                                    out.data_ptr(), pos.data_ptr(), None)
    assert rc == -5


@pytest.mark.parametrize("p", [float("inf"), 8.0])
def test_conv_layer_image_path_matches_column_path(p):
    """NormDistConv on the GPU (the kernels that work on the image, for p = inf and for finite p) against the same
    layer evaluated through F.unfold + norm_dist with autograd folding the gradient."""
    import torch.nn.functional as F
    from gpu_common import DEV, pkg
    torch.manual_seed(7)
    layer = pkg.NormDistConv(8, 12, 3, stride=1, padding=1, group=2, p=p, bias=True, mean_normalize=True).to(DEV).train()
    x = torch.randn(4, 8, 10, 10, generator=gen(56)).to(DEV)
    up = torch.randn(4, 12, 10, 10, generator=gen(57)).to(DEV)
    xa = x.clone().requires_grad_(True)
    ya, _, _ = layer(xa)
    ya.backward(up)
    ga, gwa = xa.grad.clone(), layer.weight.grad.clone()
    layer.weight.grad = None
    xb = x.clone().requires_grad_(True)
    yb = pkg.norm_dist(F.unfold(xb, 3, 1, 1, 1), layer.weight.view(12, -1), 2, p).view(4, 12, 10, 10)
    yb = layer._shift(yb)
    yb.backward(up)
    torch.cuda.synchronize()
    # p = 8: the layer runs the kernels that read the image, the comparison the column kernels (six outputs per
    # group: not even the same forward kernel); the outputs are of order 5 before the mean shift, to rel 1e-5 each
    torch.testing.assert_close(ya, yb, rtol=1e-5, atol=1e-6 if math.isinf(p) else 1e-4)
    torch.testing.assert_close(ga, xb.grad, rtol=RTOL if math.isinf(p) else 1e-4, atol=ATOL if math.isinf(p) else 1e-5)
    # p = inf: the same indices and the same upstream gradient, summed in double and rounded once on both routes;
    # p = 8: each weight gradient is a float32 sum of 400 terms of order one, in a different order per route
    if math.isinf(p):
        torch.testing.assert_close(gwa, layer.weight.grad, rtol=RTOL, atol=ATOL)
    else:
        torch.testing.assert_close(gwa, layer.weight.grad, rtol=1e-4, atol=5e-5)


BOUND_IMAGE_CASES = IMPLICIT_CASES + [(2, 96, 32, 32, 96, 1, 1, 1), (1, 192, 16, 16, 192, 1, 1, 1), (2, 96, 32, 32, 192, 1, 2, 1)]


@pytest.mark.parametrize("rows", [0, 3])
@pytest.mark.parametrize("kind", ["regular", "irregular"])
@pytest.mark.parametrize("case", BOUND_IMAGE_CASES)
def test_bound_conv_forward_matches_column_path_bit_exact(case, kind, rows):
    """Interval bounds straight from the lower and upper images against the oracle on torch's unfolded columns,
    bit for bit: regular boxes (the max3 fast path) and boxes with l > u, NaN and infinities sprinkled in, which
    send the stages that hold them through the reference's literal predicate."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, pkg, say
    B, C, H, W, CO, G, s_, p_ = case
    say("bound_conv_forward", case, kind, "rows", rows)
    lib = pkg._lib.lib()
    assert lib.ldist_set_conv_rows_override(rows) == 0
    if not cpp.inf_dist_bound_conv_forward_supported(C, H, W, CO, G, 3, s_, p_, 1):
        assert rows == 0
        pytest.skip("left to the column path by the library")
    g = gen(81)
    centre = torch.randn(B, C, H, W, generator=g)
    radius = torch.rand(B, C, H, W, generator=g) * 0.3
    lo_i, up_i = centre - radius, centre + radius
    w = torch.randn(CO, C // G * 9, generator=g) * 0.7
    if kind == "irregular":
        flat_l, flat_u = lo_i.view(-1), up_i.view(-1)
        n = flat_l.numel()
        idx = torch.randperm(n, generator=g)[: max(8, n // 500)]
        flat_l[idx[0::4]], flat_u[idx[0::4]] = flat_u[idx[0::4]].clone(), flat_l[idx[0::4]].clone()   # l > u
        flat_l[idx[1::4]] = float("nan")
        flat_u[idx[2::4]] = float("inf")
        flat_l[idx[3::4]] = -float("inf")
        w.view(-1)[5] = float("inf")
    cl = F.unfold(lo_i, 3, 1, p_, s_).contiguous()
    cu = F.unfold(up_i, 3, 1, p_, s_).contiguous()
    el, eu = oracle.inf_dist_bound_forward(cl, cu, w, G)
    ol = torch.full(el.shape, float("nan"), device=DEV)
    ou = torch.full(el.shape, float("nan"), device=DEV)
    cpp.inf_dist_bound_conv_forward(lo_i.to(DEV), up_i.to(DEV), w.to(DEV), ol, ou, G, 3, s_, p_, 1)
    torch.cuda.synchronize()
    assert torch.equal(torch.nan_to_num(ol.cpu(), nan=-7.0), torch.nan_to_num(el, nan=-7.0))
    assert torch.equal(torch.nan_to_num(ou.cpu(), nan=-7.0), torch.nan_to_num(eu, nan=-7.0))


def _misaligned(t, dev):
    """A contiguous copy of t on the device whose first element sits 4 bytes past a 16-byte boundary."""
    buf = torch.empty(t.numel() + 1, device=dev, dtype=t.dtype)
    view = buf[1:].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 16 == 4 and view.is_contiguous()
    return view


def test_conv_image_kernels_with_misaligned_tensors():
    """Every tensor 4 bytes off a 16-byte boundary: the kernels must take their scalar load and store paths
    (and the unaligned weight fetch of the argmax search) and give the same bits."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, pkg
    B, C, H, W, CO, G = 2, 8, 16, 16, 24, 2
    g = gen(91)
    img = torch.randn(B, C, H, W, generator=g)
    w = torch.randn(CO, C // G * 9, generator=g)
    cols = F.unfold(img, 3, 1, 1, 1).contiguous()
    eo, ep = oracle.inf_dist_forward(cols, w, G)
    out = _misaligned(torch.zeros(eo.shape), DEV)
    pos = _misaligned(torch.zeros(eo.shape, dtype=torch.int32), DEV)
    cpp.inf_dist_conv_forward(_misaligned(img, DEV), _misaligned(w, DEV), out, pos, G, 3, 1, 1, 1)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), eo) and torch.equal(pos.cpu(), ep)
    lo_i, up_i = img - 0.1, img + 0.1
    el, eu = oracle.inf_dist_bound_forward(F.unfold(lo_i, 3, 1, 1, 1).contiguous(), F.unfold(up_i, 3, 1, 1, 1).contiguous(),
                                           w, G)
    ol, ou = _misaligned(torch.zeros(el.shape), DEV), _misaligned(torch.zeros(el.shape), DEV)
    assert pkg._lib.lib().ldist_set_conv_rows_override(4) == 0   # a layer this small is otherwise left to the columns
    cpp.inf_dist_bound_conv_forward(_misaligned(lo_i, DEV), _misaligned(up_i, DEV), _misaligned(w, DEV), ol, ou, G, 3, 1,
                                    1, 1)
    torch.cuda.synchronize()
    assert torch.equal(ol.cpu(), el) and torch.equal(ou.cpu(), eu)
    c2 = _misaligned(torch.zeros(cols.shape), DEV)
    cpp.unfold(_misaligned(img, DEV), c2, 3, 1, 1, 1)
    gi = _misaligned(torch.zeros(img.shape), DEV)
    go = torch.randn(eo.shape, generator=g)
    cpp.inf_dist_backward_input_folded(_misaligned(go, DEV), _misaligned(ep, DEV), gi, G, 3, 1, 1, 1)
    torch.cuda.synchronize()
    assert torch.equal(c2.cpu(), cols)
    expect = F.fold(oracle.inf_dist_backward_input(go, ep, cols.size(1), G).double(), (H, W), 3, 1, 1, 1)
    torch.testing.assert_close(gi.cpu().double(), expect, rtol=RTOL, atol=1e-5)


@pytest.mark.parametrize("shape", [(40, 10, 320, 1, 1), (9, 16, 64, 2, 1), (70, 96, 260, 1, 1), (3, 12, 40, 1, 8)])
def test_column_kernels_with_misaligned_tensors(shape):
    """Every tensor 4 bytes off a 16-byte boundary: the tiled and the few-output kernels must leave their 128-bit
    load and store paths and give the same results as on aligned tensors."""
    from gpu_common import DEV, cpp
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=17 + sum(shape))
    lo, up = (x - 0.04).contiguous(), (x + 0.04).contiguous()
    eo, ep = oracle.inf_dist_forward(x, w, G)
    el, eu = oracle.inf_dist_bound_forward(lo, up, w, G)
    mis = lambda t: _misaligned(t, DEV)
    blank = lambda dtype=torch.float32: _misaligned(torch.zeros(B, CO, HW, dtype=dtype), DEV)
    xd, wd, ld, ud = mis(x), mis(w), mis(lo), mis(up)
    out, pos = blank(), blank(torch.int32)
    cpp.inf_dist_forward(xd, wd, out, pos, G)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), eo) and torch.equal(pos.cpu(), ep)
    ol, ou = blank(), blank()
    cpp.inf_dist_bound_forward(ld, ud, wd, ol, ou, G)
    torch.cuda.synchronize()
    assert torch.equal(ol.cpu(), el) and torch.equal(ou.cpu(), eu)
    ov, ol, ou = blank(), blank(), blank()
    cpp.inf_dist_value_bound_forward(xd, ld, ud, wd, ov, ol, ou, G, mis(torch.zeros(CO)), None)
    torch.cuda.synchronize()
    assert torch.equal(ov.cpu(), eo) and torch.equal(ol.cpu(), el) and torch.equal(ou.cpu(), eu)
    for p in (8.0, 150.0):
        on = blank()
        cpp.norm_dist_forward(xd, wd, on, G, p)
        torch.cuda.synchronize()
        want = oracle.norm_dist_forward(x, w, G, p)
        torch.testing.assert_close(on.cpu(), want, rtol=RTOL, atol=0)
        go = torch.randn(B, CO, HW, generator=gen(19))
        ex, mx = oracle.norm_dist_backward_input(go, x, w, want, G, p, with_abs_terms=True)
        ew, mw = oracle.norm_dist_backward_weight(go, x, w, want, G, p, with_abs_terms=True)
        gx, gw = mis(torch.zeros_like(x)), mis(torch.zeros_like(w))
        cpp.norm_dist_backward_input(mis(go), xd, wd, mis(want), gx, G, p)
        cpp.norm_dist_backward_weight(mis(go), xd, wd, mis(want), gw, G, p)
        torch.cuda.synchronize()
        assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
        assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)
    go = torch.randn(B, CO, HW, generator=gen(20))
    gx, gw = mis(torch.zeros_like(x)), mis(torch.zeros_like(w))
    cpp.inf_dist_backward_input_overwrite(mis(go), mis(ep), gx, G)
    cpp.inf_dist_backward_weight_overwrite(mis(go), mis(ep), gw, G)
    torch.cuda.synchronize()
    tx = oracle.inf_dist_backward_input(go.abs(), ep & ~SIGN, CI, G).abs()
    tw = oracle.inf_dist_backward_weight(go.abs(), ep & ~SIGN, CI, G).abs()
    assert_scatter_close(gx.cpu(), oracle.inf_dist_backward_input(go, ep, CI, G))
    assert_scatter_close(gw.cpu(), oracle.inf_dist_backward_weight(go, ep, CI, G))


def test_conv_net_runs_from_the_image_and_matches_the_column_path():
    """The reference's conv net (3 -> 32 -> 32 -> 64 -> 64 -> 64 channels at width 1) at p = inf: every conv
    layer is covered by the image kernel (resident first layer, staged wide ones, one stride-2 layer); outputs,
    input gradient and weight gradients equal those of the same net forced onto the column kernels."""
    from gpu_common import DEV, cpp, pkg
    lib = pkg._lib.lib()
    torch.manual_seed(11)
    net = pkg.Conv(width=1, input_dim=(3, 32, 32), hidden=64, num_classes=10).to(DEV).train()
    pkg.set_p_norm(net, float("inf"))
    for layer in net.conv:
        assert cpp.inf_dist_conv_forward_supported(layer.in_channels, 32 if layer.in_channels <= 32 else 16,
                                                   32 if layer.in_channels <= 32 else 16, layer.out_channels, 1, 3,
                                                   layer.stride, 1, 1)
    x = torch.rand(4, 3, 32, 32, generator=gen(71)).to(DEV)
    up = torch.randn(4, 10, generator=gen(72)).to(DEV)
    results = []
    for mode in (0, 3):                      # 0: image kernels where they apply; 3: column kernels everywhere
        assert lib.ldist_set_conv_staging_override(mode) == 0
        for prm in net.parameters():
            prm.grad = None
        for m in net.modules():              # same running means on both passes
            if isinstance(m, pkg.MeanNorm):
                m.running_mean.zero_()
        xi = x.clone().requires_grad_(True)
        y, _, _ = net(xi)
        y.backward(up)
        torch.cuda.synchronize()
        results.append((y.detach().clone(), xi.grad.clone(), [prm.grad.clone() for prm in net.parameters()]))
    lib.ldist_set_conv_staging_override(0)
    (ya, ga, wa), (yb, gb, wb) = results
    assert torch.equal(ya, yb)                                   # same argmax, same values: bit-identical forward
    torch.testing.assert_close(ga, gb, rtol=RTOL, atol=ATOL)
    for a_, b_ in zip(wa, wb):
        # the upstream gradients of the two routes differ in their last bits from the second layer down (autograd's
        # fold sums in float32), and a weight gradient sums thousands of them
        torch.testing.assert_close(a_, b_, rtol=1e-4, atol=5e-5)


def test_conv_net_certification_from_the_images_matches_the_column_path():
    """The conv net in evaluation mode with interval bounds: values and both bounds of the whole net computed
    through the image kernels are bit-identical to those through unfold + column kernels."""
    from gpu_common import DEV, pkg
    lib = pkg._lib.lib()
    torch.manual_seed(13)
    net = pkg.Conv(width=1, input_dim=(3, 32, 32), hidden=64, num_classes=10).to(DEV).eval()
    pkg.set_p_norm(net, float("inf"))
    x = torch.rand(4, 3, 32, 32, generator=gen(75)).to(DEV)
    eps = 8.0 / 255
    lower, upper = (x - eps).clamp(0, 1), (x + eps).clamp(0, 1)
    results = []
    for mode in (0, 3):
        assert lib.ldist_set_conv_staging_override(mode) == 0
        with torch.no_grad():
            results.append([t.clone() for t in net(x, lower, upper)])
    lib.ldist_set_conv_staging_override(0)
    torch.cuda.synchronize()
    for a_, b_ in zip(*results):
        assert torch.equal(a_, b_)
    y, lo, up = results[0]
    assert bool((lo <= y).all()) and bool((y <= up).all())


def test_harness_on_gpu_trains_attacks_and_certifies():
    """Model(MLP, BoundFinalIdentity): a few training steps at p = 8 lower the loss; PGD stays in its ball; the
    certified accuracy at eps = 0 equals the clean accuracy and does not grow with eps."""
    import torch.nn.functional as F
    from gpu_common import DEV, pkg
    torch.manual_seed(12)
    net = pkg.Model(pkg.MLP(depth=3, width=1, input_dim=(1, 8, 8), num_classes=4), pkg.BoundFinalIdentity(),
                    eps=0.05).to(DEV)
    pkg.set_p_norm(net, 8.0)
    x = torch.rand(64, 1, 8, 8, generator=gen(73)).to(DEV)
    y = torch.randint(0, 4, (64,), generator=gen(74)).to(DEV)
    opt = pkg.AdamW(net, lr=0.02, weight_decay=0.0)
    loss_fun = lambda out, worse, t: F.cross_entropy(out, t)
    first, _ = pkg.train_step(net, loss_fun, opt, x, y)
    for _ in range(30):
        last, _ = pkg.train_step(net, loss_fun, opt, x, y)
    assert last < first
    net.eval()
    up_, down_ = torch.ones_like(x[0]), torch.zeros_like(x[0])
    adv = pkg.AttackPGD(net, 0.05, 0.0125, 5, up_, down_).find(x, y)
    assert float((adv - x).abs().max()) <= 0.05 + 1e-6 and float(adv.min()) >= 0 and float(adv.max()) <= 1
    pkg.set_p_norm(net, float("inf"))
    with torch.no_grad():
        clean = pkg.cal_acc(net(x), y).mean().item()
    c0 = pkg.certified_accuracy(net, x, y, 0.0, up_, down_)
    c1 = pkg.certified_accuracy(net, x, y, 0.02, up_, down_)
    c2 = pkg.certified_accuracy(net, x, y, 0.2, up_, down_)
    assert abs(c0 - clean) < 1e-6 and c0 >= c1 >= c2
    assert pkg.get_p_norm(net) == float("inf") and pkg.get_eps(net) == 0.05


def test_error_codes_and_checks():
    from gpu_common import DEV, cpp, pkg
    lib = pkg._lib.lib()
    x = torch.zeros(2, 6, 1, device=DEV)
    w = torch.zeros(4, 6, device=DEV)
    out = torch.empty(2, 4, 1, device=DEV)
    pos = torch.empty(2, 4, 1, device=DEV, dtype=torch.int32)
    assert lib.ldist_inf_dist_forward(None, w.data_ptr(), 2, 4, 6, 1, 1, out.data_ptr(), pos.data_ptr(), None) == -1
    assert lib.ldist_inf_dist_forward(x.data_ptr(), w.data_ptr(), 2, 4, 6, 4, 1, out.data_ptr(), pos.data_ptr(),
                                      None) == -1  # CI % G
    assert lib.ldist_norm_dist_forward(x.data_ptr(), w.data_ptr(), 2, 4, 6, 1, 1, out.data_ptr(), 1.0, None) == -1
    with pytest.raises(RuntimeError):
        cpp.inf_dist_forward(x.cpu(), w, out, pos, 1)
    with pytest.raises(RuntimeError):
        cpp.inf_dist_forward(x, torch.zeros(6, 4, device=DEV).t(), out, pos, 1)  # weight not contiguous
    with pytest.raises(RuntimeError):
        cpp.norm_dist_forward(x, w, out, 1, 0.5)


NORM_IMAGE_CASES = [c + (1,) for c in IMPLICIT_CASES] + [  # B, C, H, W, CO, G, stride, padding, dilation
    (2, 5, 17, 17, 20, 1, 2, 0, 1),      # stride 2 without padding, odd image, odd channel count
    (2, 4, 6, 6, 24, 1, 1, 2, 1),        # padding wider than the window needs
    (2, 6, 12, 12, 20, 1, 1, 2, 2),      # dilation 2
    (2, 8, 16, 16, 40, 2, 1, 1, 1),      # two groups of 20 outputs
    (3, 8, 9, 7, 18, 1, 1, 1, 1),        # 63 positions per image: rows of a tile cross image borders, HW % 4 != 0
]


def _norm_image_problem(case, seed):
    import torch.nn.functional as F
    B, C, H, W, CO, G, s_, p_, d_ = case
    g = gen(seed)
    img = torch.rand(B, C, H, W, generator=g)
    w = torch.randn(CO, C // G * 9, generator=g) / (C // G * 9) ** 0.5
    cols = F.unfold(img, 3, d_, p_, s_).contiguous()
    go = torch.randn(B, CO, cols.size(2), generator=g)
    return img, w, cols, go


@pytest.mark.parametrize("p", [8.0, 3.0, 5.5, 100.0])
@pytest.mark.parametrize("case", NORM_IMAGE_CASES)
def test_norm_conv_forward_from_the_image(case, p):
    """p-norm forward straight from the image against the oracle on torch's unfolded columns (rel 1e-5), and
    against this library's column kernel on the same columns bit for bit where both run the tiled kernel (more
    than 16 outputs per group: the same arithmetic in the same order, only the loads differ)."""
    from gpu_common import DEV, cpp, say
    B, C, H, W, CO, G, s_, p_, d_ = case
    say("norm_conv_forward", case, "p", p)
    assert cpp.norm_dist_conv_supported(C, H, W, CO, G, 3, s_, p_, d_)
    img, w, cols, _ = _norm_image_problem(case, 91)
    want = oracle.norm_dist_forward(cols, w, G, p)
    out = torch.full(want.shape, float("nan"), device=DEV)
    cpp.norm_dist_conv_forward(img.to(DEV), w.to(DEV), out, G, p, 3, s_, p_, d_)
    from_cols = torch.full(want.shape, float("nan"), device=DEV)
    cpp.norm_dist_forward(cols.to(DEV), w.to(DEV), from_cols, G, p)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
    if CO // G > 16:
        assert torch.equal(out, from_cols)
    else:
        torch.testing.assert_close(out, from_cols, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("p", [8.0, 3.0, 5.5, 100.0])
@pytest.mark.parametrize("case", NORM_IMAGE_CASES)
def test_norm_conv_backward_from_the_image(case, p):
    """Both p-norm gradients straight from the image: grad_weight against the oracle on the unfolded columns,
    grad_img against the oracle's gradient of the columns folded back in float64 (rel 1e-5 / abs 1e-6 relative to
    the magnitude of the summed terms).  grad_img starts as NaN (the call writes every element), grad_weight at
    0.125 (the call adds)."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, say
    B, C, H, W, CO, G, s_, p_, d_ = case
    say("norm_conv_backward", case, "p", p)
    img, w, cols, go = _norm_image_problem(case, 92)
    out = oracle.norm_dist_forward(cols, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, cols, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, cols, w, out, G, p, with_abs_terms=True)
    fold = lambda t: F.fold(t.double(), (H, W), 3, d_, p_, s_)
    gi = torch.full((B, C, H, W), float("nan"), device=DEV)
    gw = torch.full((CO, C // G * 9), 0.125, device=DEV)
    args = (go.to(DEV), img.to(DEV), w.to(DEV), out.to(DEV))
    cpp.norm_dist_conv_backward_input(*args, gi, G, p, 3, s_, p_, d_)
    cpp.norm_dist_conv_backward_weight(*args, gw, G, p, 3, s_, p_, d_)
    torch.cuda.synchronize()
    assert_sum_close(gi.cpu(), fold(ex), fold(mx), p, RTOL, ATOL)
    assert_sum_close(gw.cpu() - 0.125, ew, mw, p, RTOL, ATOL)


def test_norm_conv_unsupported_geometries_are_refused():
    """Windows other than 3x3 and a single output position are left to the column kernels: the query says so and
    the entry point enqueues nothing."""
    from gpu_common import DEV, cpp, pkg
    assert not cpp.norm_dist_conv_supported(8, 16, 16, 32, 1, 5, 1, 2, 1)
    assert not cpp.norm_dist_conv_supported(8, 3, 3, 32, 1, 3, 1, 0, 1)
    assert cpp.norm_dist_conv_supported(8, 16, 16, 16, 1, 3, 1, 1, 1)
    img = torch.rand(1, 8, 3, 3, device=DEV)
    w = torch.randn(32, 72, device=DEV)
    out = torch.full((1, 32, 1), 7.0, device=DEV)
    with pytest.raises(RuntimeError):
        cpp.norm_dist_conv_forward(img, w, out, 1, 8.0, 3, 1, 0, 1)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
    del pkg


@pytest.mark.parametrize("p", [8.0, 20.0])
def test_norm_dist_conv_layer_runs_from_the_image_without_columns(p):
    """NormDistConv at finite p: same output and gradients as the layer forced through unfold + columns, and the
    peak of allocated memory stays below the size of the unfolded input (which therefore was never built)."""
    from gpu_common import DEV, cpp, pkg, say
    say("norm_dist_conv_layer", p)
    torch.manual_seed(5)
    layer = pkg.NormDistConv(128, 128, 3, padding=1, group=4, p=p, bias=True, mean_normalize=False).to(DEV)
    x = torch.rand(8, 128, 32, 32, device=DEV)
    go = torch.randn(8, 128, 32, 32, device=DEV)

    def run(force_columns):
        layer.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        layer.finite_p_route = "columns" if force_columns else "image"
        try:
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()
            y, _, _ = layer(xi)
            y.backward(go)
            torch.cuda.synchronize()
            peak = torch.cuda.max_memory_allocated() - base
        finally:
            layer.finite_p_route = "image"
        return y.detach(), xi.grad, layer.weight.grad.clone(), peak

    layer.train()
    y1, gx1, gw1, peak_img = run(False)
    y0, gx0, gw0, peak_cols = run(True)
    cols_bytes = 8 * 128 * 9 * 1024 * 4
    assert peak_img < cols_bytes <= peak_cols
    torch.testing.assert_close(y1, y0, rtol=RTOL, atol=ATOL)
    # Two float32 sums in different orders.  grad_weight adds 8192 terms of either sign per element, split over
    # workgroups that add their parts atomically in either path; the kernels' own accuracy is what the two tests
    # above check against the oracle.  A wrong tap or sign would be off by the gradient itself.  (No mean shift in
    # this layer: it centres the incoming gradient, and the terms of the -10 centre taps, all of one sign and of
    # ratio 1, then cancel to nothing, which leaves only rounding noise to compare.)
    for a, b in ((gx1, gx0), (gw1, gw0)):
        assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max())


FUSED_BACKWARD_SHAPES = [sh for sh in TILED_BACKWARD_SHAPES if sh[4] == 1] + [(515, 140, 100, 1, 1), (70, 200, 132, 1, 1)]


@pytest.mark.parametrize("tile", [0, 1, 5])
@pytest.mark.parametrize("p", [5.0, 5.5, 9.0, 20.0, 100.0, 8.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("shape", FUSED_BACKWARD_SHAPES + [(1030, 24, 44, 1, 1), (512, 64, 20, 1, 1)])
def test_norm_backward_both_gradients_in_one_pass(shape, p, tile):
    """norm_dist_backward against the oracle: the kernel that evaluates every term once for both gradients, forced
    with the tile override (by itself it only takes large layers, and p = 2 and 3 never), in its general form
    (logarithm and exponential) and its multiply-only forms for p = 2, 3, 4, 8; then override 2, which switches it
    off, so that the same call runs the two separate kernels (515 and 1030 rows, 20 and 44 columns: partial tiles of
    those).  grad_weight is added onto the buffer (0.125 here) like the separate call's."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = shape
    say("norm_backward fused", shape, "p", p, "tile", tile)
    x, w = make_inputs(B, CO, CI, G, HW, seed=36 + sum(shape))
    go = torch.randn(B, CO, HW, generator=gen(37))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    args = (go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV))
    for choice in (tile, 2):
        set_tile(choice)
        gx = torch.full((B, CI, HW), float("nan"), device=DEV)
        gw = torch.full((CO, CI // G), 0.125, device=DEV)
        cpp.norm_dist_backward(*args, gx, gw, G, p)
        torch.cuda.synchronize()
        assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
        assert_sum_close(gw.cpu() - 0.125, ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [8.0, 4.0, 20.5, 100.0])
def test_norm_backward_one_pass_on_48_column_tiles(p):
    """A layer of about 3072 inputs at batch 500: 128 x 80 and 128 x 64 tiles would leave CUs idle, so the one-call
    backward takes its 128 x 48 geometry (three columns per lane, the weight panel at a pitch of four) of its own
    accord; ragged in rows (500), outputs (260 = 4 stages of 64 + 4) and columns (3068 = 63 tiles of 48 + 44)."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = 500, 260, 3068, 1, 1
    say("norm_backward one pass, 48-column tiles", "p", p)
    set_tile(-1)
    x, w = make_inputs(B, CO, CI, G, HW, seed=61)
    go = torch.randn(B, CO, HW, generator=gen(62))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.zeros((CO, CI // G), device=DEV)
    cpp.norm_dist_backward(go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV), gx, gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [2.5, 20.0, 300.0, 8.0, 3.0])
@pytest.mark.parametrize("scale", [1e-6, 3e-4, 1.0, 5e3, 1e6, "mixed", "one tiny row"])
def test_norm_backward_both_gradients_at_every_scale(scale, p):
    """The one-call backward on inputs of every magnitude: nothing may overflow or vanish with the scale of the data
    (the one-pass kernel, forced: for a general p the power is taken of the normalised difference; at p = 3 and 8 a
    stage with an output outside [2^-12, 2^12] leaves the factored form, as in the two tiled kernels)."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = 200, 72, 132, 1, 1
    say("norm_backward fused scale", scale, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=44)
    if scale == "mixed":
        x = x * torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0])[torch.arange(B) % 5].view(B, 1, 1)
    elif scale == "one tiny row":
        x[7] *= 1e-7
    else:
        x, w = x * scale, w * scale
    x, w = x.contiguous(), w.contiguous()
    go = torch.randn(B, CO, HW, generator=gen(38))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    set_tile(0)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.zeros((CO, CI // G), device=DEV)
    cpp.norm_dist_backward(go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV), gx, gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)


ONE_PASS_EDGE_CASES = [  # B, C, H, W, CO, G, stride, padding, dilation
    (1, 4, 12, 12, 130, 1, 1, 1, 1),     # 130 outputs in one group: the LDS tiles leave room for one workgroup per CU
    (1, 4, 12, 12, 150, 1, 1, 1, 1),     # 150: the tiles do not fit, the call runs the two separate kernels
    (1, 3, 64, 64, 20, 1, 1, 1, 1),      # a tile of 64 positions is one output row: ring of four image rows, 64 wide
    (2, 9, 40, 24, 18, 1, 2, 1, 1),      # stride 2 on a 40 x 24 image: 20 x 12 positions, tiles cross output rows unevenly
    (3, 16, 5, 5, 32, 2, 1, 1, 1),       # 25 positions per image: every tile is a partial one
    (2, 7, 9, 9, 1, 1, 1, 0, 1),         # a single output
]


@pytest.mark.parametrize("p", [8.0, 5.5])
@pytest.mark.parametrize("case", ONE_PASS_EDGE_CASES)
def test_norm_conv_backward_one_pass_edge_geometries(case, p):
    """The one-pass conv backward from the image at the edges of what it takes (see the list), forced on."""
    test_norm_conv_backward_both_gradients_in_one_pass_from_the_image(case, p)


@pytest.mark.parametrize("p", [8.0, 3.0, 5.5, 100.0])
@pytest.mark.parametrize("case", NORM_IMAGE_CASES)
def test_norm_conv_backward_both_gradients_in_one_pass_from_the_image(case, p):
    """norm_dist_conv_backward on the kernel that evaluates every term once for both gradients (forced with the
    tile override; by itself it takes layers with enough rows), against the oracle on the unfolded columns, folded
    back in float64 for grad_img.  grad_img starts as NaN (the call writes every element), grad_weight at 0.125."""
    import torch.nn.functional as F
    from gpu_common import DEV, cpp, say, set_tile
    B, C, H, W, CO, G, s_, p_, d_ = case
    say("norm_conv_backward fused", case, "p", p)
    img, w, cols, go = _norm_image_problem(case, 93)
    out = oracle.norm_dist_forward(cols, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, cols, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, cols, w, out, G, p, with_abs_terms=True)
    fold = lambda t: F.fold(t.double(), (H, W), 3, d_, p_, s_)
    args = (go.to(DEV), img.to(DEV), w.to(DEV), out.to(DEV))
    for choice in (0, 2):   # one pass; the two separate kernels through the same call
        set_tile(choice)
        gi = torch.full((B, C, H, W), float("nan"), device=DEV)
        gw = torch.full((CO, C // G * 9), 0.125, device=DEV)
        cpp.norm_dist_conv_backward(*args, gi, gw, G, p, 3, s_, p_, d_)
        torch.cuda.synchronize()
        assert_sum_close(gi.cpu(), fold(ex), fold(mx), p, RTOL, ATOL)
        assert_sum_close(gw.cpu() - 0.125, ew, mw, p, RTOL, ATOL)


CONV_COLUMN_SHAPES = [sh for sh in TILED_BACKWARD_SHAPES if sh[4] > 1] + [(2, 20, 27, 1, 1024), (3, 24, 30, 2, 49)]


@pytest.mark.parametrize("p", [8.0, 2.0, 4.0, 5.5, 100.0])
@pytest.mark.parametrize("shape", CONV_COLUMN_SHAPES)
def test_norm_backward_both_gradients_in_one_pass_conv_columns(shape, p):
    """norm_dist_backward in the unfolded-conv layout on the one-pass kernel (forced with the tile override) against
    the oracle: every element of grad_input written, grad_weight added onto the buffer."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = shape
    say("norm_backward fused conv columns", shape, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=46 + sum(shape))
    go = torch.randn(B, CO, HW, generator=gen(47))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    set_tile(0)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.full((CO, CI // G), 0.125, device=DEV)
    cpp.norm_dist_backward(go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV), gx, gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu() - 0.125, ew, mw, p, RTOL, ATOL)


@pytest.mark.parametrize("p", [3.0, 8.0, 20.0])
@pytest.mark.parametrize("scale", [1e-6, 1.0, 1e6, "mixed"])
def test_norm_backward_both_gradients_conv_at_every_scale(scale, p):
    """The one-pass conv kernel where the factored form leaves the float range and a tile takes the normalised
    difference instead (images of very different magnitudes side by side)."""
    from gpu_common import DEV, cpp, say, set_tile
    B, CO, CI, G, HW = 5, 40, 36, 1, 100
    say("norm_backward fused conv scale", scale, "p", p)
    x, w = make_inputs(B, CO, CI, G, HW, seed=48)
    if scale == "mixed":
        x = x * torch.tensor([1e-5, 1.0, 1e4, 3e-3, 1.0]).view(B, 1, 1)
    else:
        x, w = x * scale, w * scale
    x, w = x.contiguous(), w.contiguous()
    go = torch.randn(B, CO, HW, generator=gen(49))
    out = oracle.norm_dist_forward(x, w, G, p)
    ex, mx = oracle.norm_dist_backward_input(go, x, w, out, G, p, with_abs_terms=True)
    ew, mw = oracle.norm_dist_backward_weight(go, x, w, out, G, p, with_abs_terms=True)
    set_tile(0)
    gx = torch.full((B, CI, HW), float("nan"), device=DEV)
    gw = torch.zeros((CO, CI // G), device=DEV)
    cpp.norm_dist_backward(go.to(DEV), x.to(DEV), w.to(DEV), out.to(DEV), gx, gw, G, p)
    torch.cuda.synchronize()
    assert_sum_close(gx.cpu(), ex, mx, p, RTOL, ATOL)
    assert_sum_close(gw.cpu(), ew, mw, p, RTOL, ATOL)


def test_fc_and_1x1_layers_accept_non_contiguous_inputs():
    """A fully connected layer and a 1x1 conv layer take a strided view as input (the reference's F.unfold always
    hands its kernels a contiguous tensor, so its layers accept such views): same output and input gradient as
    for the contiguous copy."""
    from gpu_common import DEV, pkg, say
    say("non-contiguous layer inputs")
    torch.manual_seed(11)
    fc = pkg.NormDist(24, 40, p=float("inf"), bias=True).to(DEV)
    conv = pkg.NormDistConv(6, 20, 1, p=8.0, bias=False).to(DEV)
    base_fc = torch.randn(24, 10, device=DEV)                 # (features, batch): the layer sees its transpose
    base_cv = torch.randn(5, 7, 7, 6, device=DEV)             # channels last: the layer sees a permuted view
    for layer, view in ((fc, base_fc.t()), (conv, base_cv.permute(0, 3, 1, 2))):
        assert not view.is_contiguous()
        a = view.detach().requires_grad_(True)
        b = view.detach().contiguous().requires_grad_(True)
        ya, yb = layer(a)[0], layer(b)[0]
        up = torch.randn_like(yb)
        ya.backward(up)
        yb.backward(up)
        torch.cuda.synchronize()
        assert torch.equal(ya, yb)
        assert torch.equal(a.grad, b.grad)


def test_norm_entry_points_added_to_the_abi_check_their_arguments():
    """Return codes of the entry points without a reference counterpart: null pointers and exponents that are not
    above 1 are invalid arguments, a window the image kernels do not take is 'unsupported', and in every such case
    nothing is enqueued (the outputs keep their sentinel)."""
    from gpu_common import DEV, pkg
    lib = pkg._lib.lib()
    EINVAL, EUNSUPPORTED = -1, -5
    x = torch.rand(2, 8, 1, device=DEV)
    w = torch.rand(4, 8, device=DEV)
    y = torch.rand(2, 4, 1, device=DEV) + 1
    go = torch.randn(2, 4, 1, device=DEV)
    gx = torch.full_like(x, 7.0)
    gw = torch.full_like(w, 7.0)
    P = lambda t: t.data_ptr()
    assert lib.ldist_strerror(EINVAL).startswith(b"invalid argument") and b"general path" in lib.ldist_strerror(EUNSUPPORTED)
    assert lib.ldist_norm_dist_backward(P(go), P(x), P(w), P(y), 2, 4, 8, 1, 1, P(gx), P(gw), 1.0, None) == EINVAL
    assert lib.ldist_norm_dist_backward(P(go), P(x), P(w), P(y), 2, 4, 8, 1, 1, None, P(gw), 8.0, None) == EINVAL
    assert lib.ldist_norm_dist_backward(P(go), P(x), P(w), P(y), 2, 4, 8, 3, 1, P(gx), P(gw), 8.0, None) == EINVAL   # 8 % 3
    img = torch.rand(1, 2, 6, 6, device=DEV)
    w5 = torch.rand(4, 50, device=DEV)
    y5 = torch.rand(1, 4, 4, device=DEV) + 1
    g5 = torch.randn(1, 4, 4, device=DEV)
    gi = torch.full_like(img, 7.0)
    g5w = torch.full_like(w5, 7.0)
    conv = (1, 2, 6, 6, 4, 1, 5, 5, 1, 0, 1)     # a 5x5 window
    assert lib.ldist_norm_dist_conv_supported(2, 6, 6, 4, 1, 5, 5, 1, 0, 1) == 0
    assert lib.ldist_norm_dist_conv_forward(P(img), P(w5), *conv, P(y5), 8.0, None) == EUNSUPPORTED
    assert lib.ldist_norm_dist_conv_backward(P(g5), P(img), P(w5), P(y5), *conv, P(gi), P(g5w), 8.0, None) == EUNSUPPORTED
    conv3 = (1, 2, 6, 6, 4, 1, 3, 3, 1, 1, 1)
    w3 = torch.rand(4, 18, device=DEV)
    y3 = torch.rand(1, 4, 36, device=DEV) + 1
    g3 = torch.randn(1, 4, 36, device=DEV)
    g3w = torch.full_like(w3, 7.0)
    assert lib.ldist_norm_dist_conv_backward(P(g3), P(img), P(w3), P(y3), *conv3, P(gi), P(g3w), 0.5, None) == EINVAL
    assert lib.ldist_norm_dist_conv_backward(P(g3), P(img), None, P(y3), *conv3, P(gi), P(g3w), 8.0, None) == EINVAL
    torch.cuda.synchronize()
    for t in (gx, gw, gi, g5w, g3w):
        assert bool((t == 7.0).all())
