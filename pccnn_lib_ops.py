"""``import pccnn_lib_ops`` -- the name under which the reference's Python reaches its native op module
(pccnn_lib/op_wrappers/compute_keys.py:2; built from setup.py:7-8).  With this file on the import path the 26
functions of pccnn_lib_ops/ops_list.cpp:26-54 resolve to the HIP library without any prior call."""
from pccnn_lib_amd.pccnn_lib_ops import *  # noqa: F401,F403
from pccnn_lib_amd.pccnn_lib_ops import REFERENCE_NAMES  # noqa: F401
