"""MI355X-native replacement for the per-GPU hot path of BMTrain.

Mirrors the reference's public layout for that path only:

    bmtrain_amd.C                   <- bmtrain.C            (compiled launchers)
    bmtrain_amd.optim._function     <- bmtrain.optim._function
    bmtrain_amd.optim.AdamOptimizer / AdamOffloadOptimizer / OptimManager
    bmtrain_amd.loss._function      <- bmtrain.loss._function
    bmtrain_amd.loss.FusedCrossEntropy
"""
from .global_var import config
from . import C
from . import optim
from . import loss

__all__ = ["C", "config", "optim", "loss"]
