from .cross_entropy import FusedCrossEntropy, OpFusedCrossEntropy

__all__ = ["FusedCrossEntropy", "OpFusedCrossEntropy"]
