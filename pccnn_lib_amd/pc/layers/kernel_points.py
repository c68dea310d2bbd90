"""Kernel-point layouts for KPConv.

The reference ships hard-coded layouts for K in {8, 16, 32, 64}
(pccnn_lib/pc/layers/kernel_points/kernel_points.py); this build generates its own, deterministically:
one centre point plus K - 1 points on one Fibonacci-lattice shell (K <= 16) or on two shells of radius
0.5 and 1 (K > 16).  Any K in [2, 64] is available.  A layout only has to start with the centre point:
the layer normalises it by its largest norm (pccnn_lib/pc/layers/KPConv.py:46-57)."""
import numpy as np


def _fibonacci_sphere(count):
    i = np.arange(count) + 0.5
    phi = np.arccos(1.0 - 2.0 * i / count)
    theta = np.pi * (1.0 + 5.0 ** 0.5) * i
    return np.stack([np.cos(theta) * np.sin(phi), np.sin(theta) * np.sin(phi), np.cos(phi)], axis=1)


def _circle(count, phase=0.0):
    a = 2.0 * np.pi * (np.arange(count) + phase) / max(count, 1)
    return np.stack([np.cos(a), np.sin(a)], axis=1)


def kernel_points(num_dims, num_kernel_pts):
    """A centre point plus one shell (up to 16 points) or two shells (inner one at half the radius) of evenly
    spread directions: on the unit sphere in 3 dimensions, on the unit circle in 2."""
    if num_dims not in (2, 3):
        raise RuntimeError("kernel point layouts exist for 2 and 3 dimensions only")
    if not 2 <= num_kernel_pts <= 64:
        raise RuntimeError("the number of kernel points must lie in [2, 64]")
    spread = _fibonacci_sphere if num_dims == 3 else _circle
    rest = num_kernel_pts - 1
    if num_kernel_pts <= 16:
        shell = spread(rest)
    else:
        inner = rest // 4
        shell = np.concatenate([0.5 * spread(inner), spread(rest - inner)], axis=0)
    return np.concatenate([np.zeros((1, num_dims)), shell], axis=0)


class _Layouts(dict):
    """Lookup by the reference's '<dims>_<count>' keys."""

    def __missing__(self, key):
        dims, count = key.split("_")
        self[key] = kernel_points(int(dims), int(count))
        return self[key]


kernel_pts_dict = _Layouts()
