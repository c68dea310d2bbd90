"""Model-side helpers with the reference's names (pccnn_lib/pc/models/__init__.py:1)."""
from .imodel import IModel

__all__ = ["IModel"]
