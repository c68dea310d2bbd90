"""pccnn_lib_amd: the point-cloud operator path of pccnn_lib on AMD MI355X (gfx950).

Layout (mirrors the reference's packages for this path):

* ``pccnn_lib_amd.pccnn_lib_ops``  - the native op module (same function names as the reference's
  ``pccnn_lib_ops`` extension), the compiled extension over ``libpccnn_hip.so`` when it is built, a ctypes layer otherwise
* ``pccnn_lib_amd.op_wrappers``    - torch.autograd.Function classes
* ``pccnn_lib_amd.pc``             - Pointcloud, BoundingBox, Grid, Neighborhood, PointPooling, layers, models
* ``pccnn_lib_amd.py_utils``       - host-side augmentation and sampling helpers (numpy, as in the reference)

``install_as_reference()`` registers the package under the reference's import names so that code written
against ``pccnn_lib`` / ``pccnn_lib_ops`` runs unchanged.
"""
import sys

from . import pccnn_lib_ops
from . import op_wrappers
from . import pc
from . import py_utils
from .op_wrappers import *  # noqa: F401,F403
from .pc import *  # noqa: F401,F403
from .py_utils import *  # noqa: F401,F403


def install_as_reference():
    """Make ``import pccnn_lib`` and ``import pccnn_lib_ops`` resolve to this package."""
    me = sys.modules[__name__]
    sys.modules.setdefault("pccnn_lib_ops", pccnn_lib_ops)
    sys.modules.setdefault("pccnn_lib", me)
    sys.modules.setdefault("pccnn_lib.op_wrappers", op_wrappers)
    sys.modules.setdefault("pccnn_lib.pc", pc)
    sys.modules.setdefault("pccnn_lib.pc.layers", pc.layers)
    sys.modules.setdefault("pccnn_lib.pc.models", pc.models)
    sys.modules.setdefault("pccnn_lib.py_utils", py_utils)
    return me
