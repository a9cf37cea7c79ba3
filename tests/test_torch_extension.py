"""The PyTorch-ROCm C++ extension `norm_dist_cpp` (l_inf-dist-net_amd/csrc/torch_ext/norm_dist_cpp.cpp): the module
name and the seven functions the reference's model/norm_dist.py imports (reference model/norm_dist.cpp:92-100), as a
pybind11 layer over the C ABI.  Without a GPU: it loads, exports exactly those names, and rejects tensors the way the
reference's checks do.  With one: every function gives the bits the ctypes binding gives (both call the same library),
on the caller's current stream."""
import pytest
import torch

import __graft_entry__ as entry
from helpers import gen, make_inputs

pkg = entry.load_package()
cpp = pkg.norm_dist_cpp

SEVEN = ["inf_dist_backward_input", "inf_dist_backward_weight", "inf_dist_bound_forward", "inf_dist_forward",
         "norm_dist_backward_input", "norm_dist_backward_weight", "norm_dist_forward"]


def _ext():
    ext = cpp.torch_extension()
    if ext is None:
        pytest.skip("torch_ext/norm_dist_cpp*.so has not been built (make -C l_inf-dist-net_amd/csrc torch_ext)")
    return ext


def test_extension_exports_the_reference_module():
    ext = _ext()
    assert ext.__name__ == "norm_dist_cpp"
    assert sorted(n for n in dir(ext) if not n.startswith("_")) == SEVEN          # model/norm_dist.cpp:92-100
    assert sorted(cpp.REFERENCE_NAMES) == SEVEN
    # built => the package's autograd functions go through it; the ctypes functions stay reachable
    assert cpp.BINDING == "torch_extension" and cpp.inf_dist_forward is ext.inf_dist_forward
    assert cpp.use_torch_extension(False) == "ctypes" and cpp.inf_dist_forward is cpp.ctypes_binding["inf_dist_forward"]
    assert cpp.use_torch_extension(True) == "torch_extension"


def test_extension_rejects_what_the_reference_rejects():
    ext = _ext()
    x, w = torch.zeros(2, 4, 1), torch.zeros(3, 4)
    out, pos = torch.zeros(2, 3, 1), torch.zeros(2, 3, 1, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):              # CHECK_CUDA, model/norm_dist.cpp:3
        ext.inf_dist_forward(x, w, out, pos, 1)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.norm_dist_backward_weight(out, x, w, out, w, 1, 8.0)
    with pytest.raises(TypeError):                                                # positional signature of the reference
        ext.inf_dist_forward(x, w, out, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(6, 24, 40, 1, 1), (3, 8, 12, 2, 5), (64, 96, 256, 1, 1)])
def test_extension_matches_the_ctypes_binding_bit_for_bit(shape):
    ext = _ext()
    dev = torch.device("cuda:0")
    B, CO, CI, G, HW = shape
    x, w = make_inputs(B, CO, CI, G, HW, seed=91)
    xd, wd = x.to(dev), w.to(dev)
    go = torch.randn(B, CO, HW, generator=gen(92)).to(dev)
    ct = cpp.ctypes_binding

    def both(name, make_outputs, args_before, args_after):
        res = []
        for fn in (getattr(ext, name), ct[name]):
            outs = make_outputs()
            fn(*args_before, *outs, *args_after)
            torch.cuda.synchronize()
            res.append(outs)
        for a, b in zip(*res):
            assert torch.equal(a, b), name
        return res[0]

    new = lambda dt=torch.float32: torch.empty(B, CO, HW, device=dev, dtype=dt)
    out, pos = both("inf_dist_forward", lambda: [new(), new(torch.int32)], (xd, wd), (G,))
    both("inf_dist_bound_forward", lambda: [new(), new()], ((xd - 0.1).contiguous(), (xd + 0.1).contiguous(), wd), (G,))
    both("inf_dist_backward_input", lambda: [torch.zeros_like(xd)], (go, pos), (G,))
    both("inf_dist_backward_weight", lambda: [torch.zeros_like(wd)], (go, pos), (G,))
    (o8,) = both("norm_dist_forward", lambda: [new()], (xd, wd), (G, 8.0))
    both("norm_dist_backward_input", lambda: [torch.empty_like(xd)], (go, xd, wd, o8), (G, 8.0))
    both("norm_dist_backward_weight", lambda: [torch.zeros_like(wd)], (go, xd, wd, o8), (G, 8.0))
    # non-contiguous and wrong-dtype tensors on the GPU, and a shape the operator cannot take
    with pytest.raises(RuntimeError, match="must be contiguous"):                 # CHECK_CONTIGUOUS, model/norm_dist.cpp:4
        ext.inf_dist_forward(xd.transpose(0, 1), wd, out, pos, G)
    with pytest.raises(RuntimeError, match="int32"):
        ext.inf_dist_forward(xd, wd, out, out, G)
    with pytest.raises(RuntimeError, match="group"):
        ext.inf_dist_forward(xd, wd[:, :-1].contiguous(), out, pos, G)


@pytest.mark.gpu
def test_extension_launches_on_the_current_stream():
    """A side stream that first waits on a long-running kernel: the extension's result must come after it, i.e. the
    call went to that stream and not to the default one (the reference launches on the legacy default stream)."""
    ext = _ext()
    dev = torch.device("cuda:0")
    x, w = make_inputs(32, 64, 128, 1, 1, seed=93)
    xd, wd = x.to(dev), w.to(dev)
    out = torch.empty(32, 64, 1, device=dev)
    pos = torch.empty(32, 64, 1, device=dev, dtype=torch.int32)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        filler = torch.zeros(64 << 20, device=dev)
        for _ in range(20):
            filler.add_(1.0)                       # some milliseconds of work queued on the side stream
        xs = xd + filler[:1].sum() * 0.0 + 1.0     # produced on the side stream, after the filler
        ext.inf_dist_forward(xs.contiguous(), wd, out, pos, 1)
    side.synchronize()
    want, _ = (t.clone() for t in (out, pos))
    ref = torch.empty_like(out)
    cpp.ctypes_binding["inf_dist_forward"]((xd + 1.0).contiguous(), wd, ref, pos, 1)
    torch.cuda.synchronize()
    assert torch.equal(want, ref)
