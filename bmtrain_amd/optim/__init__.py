from .adam import AdamOptimizer
from .adam_offload import AdamOffloadOptimizer
from .optim_manager import OptimManager

__all__ = ["AdamOptimizer", "AdamOffloadOptimizer", "OptimManager"]
