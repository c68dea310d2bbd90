"""torch.autograd.Function wrappers of the native ops, same class names, argument order and
gradient routing as the reference's pccnn_lib/op_wrappers package."""
from .index_ops import BuildGridDS, ComputeKeys, FindNeighbors, PoissonDiskSamlping
from .density import ComputePDF
from .convolutions import (ComputeKPConv, ComputeKPConvWeightVar, ComputeMCConv, ComputeMCConvWeightVar,
                           ComputePointConvBasis, ComputePointConv, ComputePointConvWeightVar, ComputeKPConvN,
                           ComputeKPConvNWeightVar, ComputeSPHConv, ComputeSPHConvWeightVar, ComputePCCNN,
                           ComputePCCNNWeightVar)

__all__ = ["BuildGridDS", "ComputeKeys", "FindNeighbors", "PoissonDiskSamlping", "ComputePDF",
           "ComputeKPConv", "ComputeKPConvWeightVar", "ComputeMCConv", "ComputeMCConvWeightVar",
           "ComputePointConvBasis", "ComputePointConv", "ComputePointConvWeightVar",
           "ComputeKPConvN", "ComputeKPConvNWeightVar", "ComputeSPHConv", "ComputeSPHConvWeightVar",
           "ComputePCCNN", "ComputePCCNNWeightVar"]
