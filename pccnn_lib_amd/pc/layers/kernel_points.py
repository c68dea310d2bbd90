"""Kernel-point layouts for KPConv.

The reference's twelve constant layouts (2, 3 and 4 dimensions, K in {8, 16, 32, 64};
pccnn_lib/pc/layers/kernel_points/kernel_points.py:3-364) are read from ``kernel_points_tables.txt`` beside this file,
so a layer built for one of those keys has the reference's ``kernel_pts_`` and ``sigma_``.  Any other key
(2 to 6 dimensions, K in [2, 64], e.g. the 15 points of ``3_15``) is generated deterministically: one centre point plus
K - 1 points on one shell (K <= 16) or on two shells of radius 0.5 and 1 (K > 16).  A layout only has to start with the
centre point: the layer normalises it by its largest norm (pccnn_lib/pc/layers/KPConv.py:46-57)."""
import os

import numpy as np

TABLES_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_points_tables.txt")


def load_tables(path=TABLES_PATH):
    """{'<dims>_<count>': float64 [count, dims]} from the data file: a line 'dims count', then the rows."""
    tables = {}
    with open(path) as handle:
        lines = [l.split() for l in handle if l.strip() and not l.startswith("#")]
    pos = 0
    while pos < len(lines):
        dims, count = int(lines[pos][0]), int(lines[pos][1])
        block = np.array(lines[pos + 1:pos + 1 + count], dtype=np.float64)
        if block.shape != (count, dims):
            raise RuntimeError("kernel point table %d_%d is malformed in %s" % (dims, count, path))
        tables["%d_%d" % (dims, count)] = block
        pos += 1 + count
    return tables


def _fibonacci_sphere(count):
    i = np.arange(count) + 0.5
    phi = np.arccos(1.0 - 2.0 * i / count)
    theta = np.pi * (1.0 + 5.0 ** 0.5) * i
    return np.stack([np.cos(theta) * np.sin(phi), np.sin(theta) * np.sin(phi), np.cos(phi)], axis=1)


def _circle(count, phase=0.0):
    a = 2.0 * np.pi * (np.arange(count) + phase) / max(count, 1)
    return np.stack([np.cos(a), np.sin(a)], axis=1)


def _hypersphere(num_dims, count):
    """`count` directions spread over the unit sphere of `num_dims` >= 4 dimensions: a low-discrepancy sequence
    (additive recurrence on the roots of x^(n+1) = x + 1) pushed through Box-Muller and normalised, then evened out by
    a fixed number of repulsion steps along the sphere.  Deterministic: no random numbers."""
    if count == 0:
        return np.zeros((0, num_dims))
    cols = 2 * ((num_dims + 1) // 2)
    g = 2.0
    for _ in range(64):
        g = (1.0 + g) ** (1.0 / (cols + 1))
    alpha = (1.0 / g) ** np.arange(1, cols + 1)
    u = np.mod(0.5 + np.outer(np.arange(1, count + 1), alpha), 1.0)
    r = np.sqrt(-2.0 * np.log(np.maximum(u[:, 0::2], 1e-12)))
    a = 2.0 * np.pi * u[:, 1::2]
    x = np.concatenate([r * np.cos(a), r * np.sin(a)], axis=1)[:, :num_dims]
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    for step in range(200):
        diff = x[:, None, :] - x[None, :, :]
        dist2 = np.sum(diff * diff, axis=-1) + np.eye(count)
        force = np.sum(diff / dist2[..., None] ** 1.5, axis=1)
        force -= np.sum(force * x, axis=1, keepdims=True) * x          # keep the step on the sphere
        norm = np.linalg.norm(force, axis=1, keepdims=True)
        x = x + 0.1 * (0.98 ** step) * force / np.maximum(norm.max(), 1e-12)
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    return x


def kernel_points(num_dims, num_kernel_pts):
    """A centre point plus one shell (up to 16 points) or two shells (inner one at half the radius) of evenly
    spread directions: on the unit circle in 2 dimensions, the unit sphere in 3, the unit hypersphere beyond."""
    if not 2 <= num_dims <= 6:
        raise RuntimeError("kernel point layouts exist for 2 to 6 dimensions")
    if not 2 <= num_kernel_pts <= 64:
        raise RuntimeError("the number of kernel points must lie in [2, 64]")
    if num_dims == 2:
        spread = _circle
    elif num_dims == 3:
        spread = _fibonacci_sphere
    else:
        spread = lambda count: _hypersphere(num_dims, count)
    rest = num_kernel_pts - 1
    if num_kernel_pts <= 16:
        shell = spread(rest)
    else:
        inner = rest // 4
        shell = np.concatenate([0.5 * spread(inner), spread(rest - inner)], axis=0)
    return np.concatenate([np.zeros((1, num_dims)), shell], axis=0)


class _Layouts(dict):
    """Lookup by the reference's '<dims>_<count>' keys: the constant tables, else a generated layout."""

    def __missing__(self, key):
        dims, count = key.split("_")
        self[key] = kernel_points(int(dims), int(count))
        return self[key]


kernel_pts_dict = _Layouts(load_tables())
