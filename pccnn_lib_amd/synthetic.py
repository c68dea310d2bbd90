"""Seeded synthetic point clouds for tests and the benchmark (numpy, host side).

* ``sphere_surface`` follows pccnn_lib/py_utils/pc_utils.py:128-141 (normalised Gaussian draws).
* ``primitives`` draws area-uniform surface samples of a sphere, box, cylinder or torus, rotates
  them randomly and scales them into the unit cube.
* ``room`` is a 10 x 10 x 3 m room (floor, ceiling, four walls) with axis-aligned boxes inside,
  sampled with area-weighted uniform density plus Gaussian jitter.
"""
import numpy as np


def sphere_surface(rng, num_pts, num_dims=3):
    pts = rng.normal(0.0, 1.0, (num_pts, num_dims))
    pts = pts / np.linalg.norm(pts, axis=1)[:, None]
    return pts.astype(np.float32)


def _random_rotation(rng):
    q, r = np.linalg.qr(rng.normal(size=(3, 3)))
    q = q * np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q


def _box_surface(rng, n, half):
    hx, hy, hz = half
    areas = np.array([hy * hz, hy * hz, hx * hz, hx * hz, hx * hy, hx * hy])
    face = rng.choice(6, size=n, p=areas / areas.sum())
    u = rng.uniform(-1, 1, (n, 3)) * np.asarray(half)
    axis = face // 2
    sign = np.where(face % 2 == 0, -1.0, 1.0)
    u[np.arange(n), axis] = sign * np.asarray(half)[axis]
    return u


def _primitive(rng, kind, n):
    if kind == 0:                                   # sphere
        return sphere_surface(rng, n).astype(np.float64)
    if kind == 1:                                   # box
        return _box_surface(rng, n, rng.uniform(0.4, 1.0, 3))
    if kind == 2:                                   # cylinder (side + caps)
        r, h = rng.uniform(0.4, 1.0), rng.uniform(0.5, 1.5)
        a_side, a_cap = 2 * np.pi * r * h, np.pi * r * r
        part = rng.choice(3, size=n, p=np.array([a_side, a_cap, a_cap]) / (a_side + 2 * a_cap))
        th = rng.uniform(0, 2 * np.pi, n)
        rad = np.where(part == 0, r, r * np.sqrt(rng.uniform(0, 1, n)))
        z = np.where(part == 0, rng.uniform(-h / 2, h / 2, n), np.where(part == 1, -h / 2, h / 2))
        return np.stack([rad * np.cos(th), rad * np.sin(th), z], axis=1)
    # torus: rejection sampling for area-uniform density
    R, r = 1.0, rng.uniform(0.2, 0.45)
    out = np.zeros((0, 3))
    while out.shape[0] < n:
        u = rng.uniform(0, 2 * np.pi, 2 * n)
        v = rng.uniform(0, 2 * np.pi, 2 * n)
        keep = rng.uniform(0, 1, 2 * n) < (R + r * np.cos(v)) / (R + r)
        u, v = u[keep], v[keep]
        p = np.stack([(R + r * np.cos(v)) * np.cos(u), (R + r * np.cos(v)) * np.sin(u), r * np.sin(v)], axis=1)
        out = np.concatenate([out, p], axis=0)
    return out[:n]


def primitives(seed, batch, num_pts):
    """``batch`` clouds of ``num_pts`` surface points, each scaled into [0,1]^3.
    Returns (pts float32 [batch*num_pts, 3], batch_ids int32)."""
    rng = np.random.default_rng(seed)
    clouds = []
    for _ in range(batch):
        p = _primitive(rng, int(rng.integers(0, 4)), num_pts) @ _random_rotation(rng).T
        mn, mx = p.min(axis=0), p.max(axis=0)
        p = (p - mn) / (mx - mn).max()
        clouds.append(p.astype(np.float32))
    pts = np.concatenate(clouds, axis=0)
    ids = np.repeat(np.arange(batch, dtype=np.int32), num_pts)
    return pts, ids


def room(seed, num_pts, num_boxes=40, jitter=0.002, size=(10.0, 10.0, 3.0)):
    """One synthetic room of ``num_pts`` points (metres).  Returns float32 [num_pts, 3]."""
    rng = np.random.default_rng(seed)
    sx, sy, sz = size
    rects = []                                       # (origin, edge_u, edge_v)
    o = np.zeros(3)
    rects += [(o, [sx, 0, 0], [0, sy, 0]), (np.array([0, 0, sz]), [sx, 0, 0], [0, sy, 0]),
              (o, [sx, 0, 0], [0, 0, sz]), (np.array([0, sy, 0]), [sx, 0, 0], [0, 0, sz]),
              (o, [0, sy, 0], [0, 0, sz]), (np.array([sx, 0, 0]), [0, sy, 0], [0, 0, sz])]
    for _ in range(num_boxes):
        ext = rng.uniform(0.3, 1.5, 3)
        ext[2] = min(ext[2], sz)
        org = np.array([rng.uniform(0, sx - ext[0]), rng.uniform(0, sy - ext[1]), 0.0])
        ex, ey, ez = [ext[0], 0, 0], [0, ext[1], 0], [0, 0, ext[2]]
        rects += [(org, ex, ey), (org + ez, ex, ey), (org, ex, ez), (org + ey, ex, ez),
                  (org, ey, ez), (org + ex, ey, ez)]
    areas = np.array([np.linalg.norm(np.cross(u, v)) for _, u, v in rects])
    which = rng.choice(len(rects), size=num_pts, p=areas / areas.sum())
    org = np.array([r[0] for r in rects])[which]
    eu = np.array([r[1] for r in rects], dtype=np.float64)[which]
    ev = np.array([r[2] for r in rects], dtype=np.float64)[which]
    a, b = rng.uniform(0, 1, (num_pts, 1)), rng.uniform(0, 1, (num_pts, 1))
    pts = org + a * eu + b * ev + rng.normal(0.0, jitter, (num_pts, 3))
    return pts.astype(np.float32)


def kernel_points_sphere(seed, num_kernel_pts):
    """One centre point plus ``num_kernel_pts - 1`` seeded points on the unit sphere, normalised
    the way pccnn_lib/pc/layers/KPConv.py:46-57 normalises a layout.
    Returns (kernel_pts float32 [K,3], sigma float)."""
    rng = np.random.default_rng(seed)
    kp = np.concatenate([np.zeros((1, 3)), sphere_surface(rng, num_kernel_pts - 1).astype(np.float64)], axis=0)
    kp = kp.astype(np.float32)
    dist = np.linalg.norm(kp, axis=-1).astype(np.float32)
    max_d = dist.max()
    dist, kp = dist / max_d, kp / max_d
    min_d = dist[1:].min()
    return (kp / (1.0 + min_d)).astype(np.float32), float(min_d / (1.0 + min_d))
