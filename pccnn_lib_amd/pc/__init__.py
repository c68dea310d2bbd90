"""Point-cloud objects with the reference's names and attributes (pccnn_lib/pc/__init__.py:1-7)."""
from .point_cloud import Pointcloud
from .bounding_box import BoundingBox
from .grid import Grid
from .neighborhood import Neighborhood
from .point_pooling import PointPooling
from . import layers
from .layers import *  # noqa: F401,F403
from .layers import __all__ as _layer_names
from . import models
from .models import IModel

__all__ = ["Pointcloud", "BoundingBox", "Grid", "Neighborhood", "PointPooling", "layers", "models", "IModel"] + list(_layer_names)
