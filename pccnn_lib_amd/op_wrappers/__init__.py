"""torch.autograd.Function wrappers of the native ops, same class names, argument order and
gradient routing as the reference's pccnn_lib/op_wrappers package."""
from .index_ops import BuildGridDS, ComputeKeys, FindNeighbors, PoissonDiskSamlping
from .density import ComputePDF
from .kpconv import ComputeKPConv, ComputeKPConvWeightVar
from .mcconv import ComputeMCConv, ComputeMCConvWeightVar

__all__ = ["BuildGridDS", "ComputeKeys", "FindNeighbors", "PoissonDiskSamlping", "ComputePDF",
           "ComputeKPConv", "ComputeKPConvWeightVar", "ComputeMCConv", "ComputeMCConvWeightVar"]
