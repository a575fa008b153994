from .cross_entropy import FusedCrossEntropy, OpFusedCrossEntropy, VPFusedCrossEntropy

__all__ = ["FusedCrossEntropy", "OpFusedCrossEntropy", "VPFusedCrossEntropy"]
