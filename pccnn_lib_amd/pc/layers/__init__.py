from .norm import Bias, GroupNormalization
from .conv_base import IConvLayer, IConvLayerFactory
from .mcconv import MCConv, MCConvFactory
from .pointconv import PointConv, PointConvFactory
from .kpconv import KPConv, KPConvFactory, KPConvN, KPConvNFactory, PCCNN, PCCNNFactory
from .sphconv import SPHConv, SPHConvFactory

__all__ = ["Bias", "GroupNormalization", "IConvLayer", "IConvLayerFactory", "MCConv", "MCConvFactory", "PointConv",
           "PointConvFactory", "KPConv", "KPConvFactory", "KPConvN", "KPConvNFactory", "SPHConv", "SPHConvFactory",
           "PCCNN", "PCCNNFactory"]
