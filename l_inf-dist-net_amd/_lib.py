"""Loader for libldist_hip.so, the C-ABI library declared in include/ldist.h.

There is no fallback: if the library has not been built, or a call returns an
error code, a RuntimeError says so.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libldist_hip.so")

_F = ctypes.c_void_p   # const float* / float* (device)
_I = ctypes.c_void_p   # const int32_t* / int32_t* (device)
_S = ctypes.c_void_p   # hipStream_t
_i = ctypes.c_int
_f = ctypes.c_float
_d = ctypes.c_double

# name -> argument types, in the order of include/ldist.h
SIGNATURES = {
    "ldist_inf_dist_forward": [_F, _F, _i, _i, _i, _i, _i, _F, _I, _S],
    "ldist_inf_dist_forward_values": [_F, _F, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_bound_forward": [_F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _S],
    "ldist_inf_dist_value_bound_forward": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _F, _F, _F, _S],
    "ldist_inf_dist_backward_input": [_F, _I, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_backward_weight": [_F, _I, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_backward_input_overwrite": [_F, _I, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_backward_weight_overwrite": [_F, _I, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_backward_overwrite": [_F, _I, _i, _i, _i, _i, _i, _F, _F, _S],
    "ldist_norm_dist_forward": [_F, _F, _i, _i, _i, _i, _i, _F, _f, _S],
    "ldist_norm_dist_backward_input": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _F, _f, _S],
    "ldist_norm_dist_backward_weight": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _F, _f, _S],
    "ldist_norm_dist_backward": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _f, _S],
    "ldist_mean_shift": [_F, _i, _i, _i, _F, _F, _F, _f, _S],
    "ldist_unfold": [_F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_conv_forward_supported": [_i, _i, _i, _i, _i, _i, _i, _i, _i, _i],
    "ldist_inf_dist_conv_forward": [_F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _I, _S],
    "ldist_inf_dist_conv_forward_values": [_F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_bound_conv_forward_supported": [_i, _i, _i, _i, _i, _i, _i, _i, _i, _i],
    "ldist_inf_dist_bound_conv_forward": [_F, _F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _F, _S],
    "ldist_norm_dist_conv_supported": [_i, _i, _i, _i, _i, _i, _i, _i, _i, _i],
    "ldist_norm_dist_conv_forward": [_F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _f, _S],
    "ldist_norm_dist_conv_backward_input": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _f, _S],
    "ldist_norm_dist_conv_backward_weight": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _f, _S],
    "ldist_norm_dist_conv_backward": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _F, _f, _S],
    "ldist_fold": [_F, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _S],
    "ldist_inf_dist_backward_input_folded": [_F, _I, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _F, _S],
    "ldist_adamw_lp_step": [_F, _F, _F, _F, _i, _i, _d, _d, _d, _d, _d, _d, _i, _S],
}

_lib = None


def build():
    """Compile the library in-tree with hipcc (gfx950).  Needs no GPU."""
    import subprocess
    subprocess.run(["make", "-s", "-j8", "-C", os.path.join(_HERE, "csrc")], check=True)
    subprocess.run(["make", "-s", "-C", os.path.join(_HERE, "csrc"), "torch_ext"], check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(or __graft_entry__.build()); the distance-neuron operators have no other backend")
        handle = ctypes.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = args
            fn.restype = ctypes.c_int
        handle.ldist_set_tile_override.argtypes = [ctypes.c_int]
        handle.ldist_set_tile_override.restype = ctypes.c_int
        handle.ldist_set_conv_rows_override.argtypes = [ctypes.c_int]
        handle.ldist_set_conv_rows_override.restype = ctypes.c_int
        handle.ldist_set_conv_staging_override.argtypes = [ctypes.c_int]
        handle.ldist_set_conv_staging_override.restype = ctypes.c_int
        handle.ldist_version.restype = ctypes.c_int
        handle.ldist_strerror.restype = ctypes.c_char_p
        handle.ldist_strerror.argtypes = [ctypes.c_int]
        handle.ldist_last_hip_error.restype = ctypes.c_int
        _lib = handle
    return _lib


EUNSUPPORTED = -5   # LDIST_EUNSUPPORTED of include/ldist.h: a specialised entry point does not cover the problem


def check(rc, name):
    if rc != 0:
        handle = lib()
        msg = handle.ldist_strerror(rc).decode()
        extra = f" (hipError_t {handle.ldist_last_hip_error()})" if rc == -3 else ""
        raise RuntimeError(f"{name} failed: {msg}{extra}")
