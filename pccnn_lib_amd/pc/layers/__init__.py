"""The layer classes and their factories under the reference's names (pccnn_lib/pc/layers/__init__.py:1-10); several of
them share a module here."""
import importlib

_HOMES = {
    "norm": ("Bias", "GroupNormalization"),
    "conv_base": ("IConvLayer", "IConvLayerFactory"),
    "mcconv": ("MCConv", "MCConvFactory"),
    "pointconv": ("PointConv", "PointConvFactory"),
    "kpconv": ("KPConv", "KPConvFactory", "KPConvN", "KPConvNFactory", "PCCNN", "PCCNNFactory"),
    "sphconv": ("SPHConv", "SPHConvFactory"),
}

__all__ = []
for _home, _names in _HOMES.items():
    _module = importlib.import_module("." + _home, __name__)
    for _name in _names:
        globals()[_name] = getattr(_module, _name)
        __all__.append(_name)
del _home, _names, _module, _name
