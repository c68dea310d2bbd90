"""Point-cloud objects with the reference's names and attributes (pccnn_lib/pc/__init__.py:1-5)."""
from .point_cloud import Pointcloud
from .bounding_box import BoundingBox
from .grid import Grid
from .neighborhood import Neighborhood
from .point_pooling import PointPooling
from . import layers
from .layers import IConvLayer, IConvLayerFactory, KPConv, KPConvFactory, MCConv, MCConvFactory

__all__ = ["Pointcloud", "BoundingBox", "Grid", "Neighborhood", "PointPooling", "layers", "IConvLayer",
           "IConvLayerFactory", "KPConv", "KPConvFactory", "MCConv", "MCConvFactory"]
