from .conv_base import IConvLayer, IConvLayerFactory
from .kpconv import KPConv, KPConvFactory
from .mcconv import MCConv, MCConvFactory

__all__ = ["IConvLayer", "IConvLayerFactory", "KPConv", "KPConvFactory", "MCConv", "MCConvFactory"]
