"""torch.autograd.Function wrappers of the native ops, same class names, argument order and
gradient routing as the reference's pccnn_lib/op_wrappers package."""
from .index_ops import BuildGridDS, ComputeKeys, FindNeighbors, PoissonDiskSamlping
from .density import ComputePDF
from .kpconv import ComputeKPConv, ComputeKPConvWeightVar
from .mcconv import ComputeMCConv, ComputeMCConvWeightVar
from .pointconv import ComputePointConvBasis, ComputePointConv, ComputePointConvWeightVar
from .kpconvn import ComputeKPConvN, ComputeKPConvNWeightVar
from .sphconv import ComputeSPHConv, ComputeSPHConvWeightVar
from .pccnn import ComputePCCNN, ComputePCCNNWeightVar

__all__ = ["BuildGridDS", "ComputeKeys", "FindNeighbors", "PoissonDiskSamlping", "ComputePDF",
           "ComputeKPConv", "ComputeKPConvWeightVar", "ComputeMCConv", "ComputeMCConvWeightVar",
           "ComputePointConvBasis", "ComputePointConv", "ComputePointConvWeightVar",
           "ComputeKPConvN", "ComputeKPConvNWeightVar", "ComputeSPHConv", "ComputeSPHConvWeightVar",
           "ComputePCCNN", "ComputePCCNNWeightVar"]
