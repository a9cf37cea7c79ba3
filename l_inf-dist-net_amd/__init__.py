"""MI355X-native L_p / L_inf distance-neuron operators (gfx950 HIP kernels behind a C ABI).

Python surface = the reference's model/norm_dist.py (plus its optimizer, adamw.py); native surface = include/ldist.h.
"""
from . import norm_dist_cpp
from .adamw import AdamW, lp_weight_decay_
from ._lib import LIB_PATH, build as build_library
from .conv import Conv
from .harness import AttackPGD, Model, cal_acc, certified_accuracy, get_eps, set_eps, train_step
from .mlp import MLP, BoundFinalIdentity
from .norm_dist import (DistF, MeanNorm, MeanNormDist, NormDist, NormDistConv, get_p_norm, inf_dist_bound, norm_dist,
                        set_p_norm)

__all__ = ["DistF", "MeanNorm", "MeanNormDist", "NormDist", "NormDistConv", "get_p_norm", "set_p_norm", "norm_dist",
           "inf_dist_bound", "norm_dist_cpp", "MLP", "BoundFinalIdentity", "Conv", "Model", "AttackPGD", "certified_accuracy", "train_step", "cal_acc",
           "set_eps", "get_eps", "AdamW", "lp_weight_decay_", "LIB_PATH", "build_library"]
