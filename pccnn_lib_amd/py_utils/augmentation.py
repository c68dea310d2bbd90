"""Data augmentation and small-scale sampling on the host, in numpy (the interface of pccnn_lib/py_utils/pc_utils.py).

These run before a cloud reaches the GPU and are numpy code in the reference too.  Every function that takes a
``numpy.random.RandomState`` draws from it in the reference's order and with the reference's shapes, so a script that
seeds its state gets the same augmented clouds from either package."""
import numpy as np


def jitter_pc(p_random_state, p_pts, p_noise=0.001, p_clip=0.005):
    """Gaussian noise of standard deviation ``p_noise`` on every coordinate, limited to +-``p_clip`` when that is
    positive (pc_utils.py:3-20).  One ``randn(n, d)`` draw."""
    noise = p_random_state.randn(*p_pts.shape[:2]) * p_noise
    if p_clip > 0.0:
        noise = np.clip(noise, -1.0 * p_clip, p_clip)
    return p_pts + noise


def mirror_pc(p_random_state, p_axis, p_pts, p_normals=None, p_return_mirror=False):
    """Flip the sign of each axis allowed in ``p_axis`` with probability one half (pc_utils.py:23-47).  One
    ``random_sample()`` draw per entry of ``p_axis``, allowed or not.  Returns (points, normals or None) and, when
    asked, the float32 [1, d] vector of signs as a third value."""
    signs = np.ones((1, p_pts.shape[1]), dtype=np.float32)
    for axis, allowed in enumerate(p_axis):
        flip = p_random_state.random_sample() > 0.5
        if flip and allowed:
            signs[0, axis] = -1.0
    normals = None if p_normals is None else p_normals * signs
    if p_return_mirror:
        return p_pts * signs, normals, signs
    return p_pts * signs, normals


def anisotropic_scale_pc(p_random_state, p_pts, p_min_scale=0.9, p_max_scale=1.1, p_return_scaling=False):
    """One scale factor per axis, uniform in [p_min_scale, p_max_scale) (pc_utils.py:50-74): a single
    ``random_sample((1, d))`` draw."""
    factors = p_random_state.random_sample((1, p_pts.shape[1])) * (p_max_scale - p_min_scale) + p_min_scale
    if p_return_scaling:
        return p_pts * factors, factors
    return p_pts * factors


def _axis_rotation(axis, angle):
    """Right-handed rotation by ``angle`` about coordinate axis 0, 1 or 2 (float64 3 x 3)."""
    c, s = np.cos(angle), np.sin(angle)
    i, j = ((1, 2), (2, 0), (0, 1))[axis]
    m = np.eye(3)
    m[i, i], m[i, j], m[j, i], m[j, j] = c, -s, s, c
    return m


def rotate_pc_3d(p_random_state, p_pts, p_max_angle=2.0 * np.pi, p_axes=(0, 1, 2)):
    """Random rotation of a 3-D cloud (pc_utils.py:77-125): three angles uniform in +-``p_max_angle`` from one
    ``random_sample(3)`` draw (all three are drawn whichever axes are enabled), R = Rz Ry Rx over the axes listed in
    ``p_axes``, points multiplied from the left (``pts @ R``).  Returns (rotated points, R)."""
    angles = (p_random_state.random_sample((3)) - 0.5) * 2.0 * p_max_angle
    rx, ry, rz = [_axis_rotation(a, angles[a]) if a in p_axes else np.eye(3) for a in range(3)]
    rotation = np.dot(rz, np.dot(ry, rx))
    return np.dot(p_pts, rotation), rotation


def uniform_samples_surface_sphere(p_random_state, p_num_pts, p_num_dims):
    """``p_num_pts`` points uniform on the unit sphere in ``p_num_dims`` dimensions: normalised Gaussian vectors,
    float32 (pc_utils.py:128-141)."""
    pts = p_random_state.normal(0.0, 1.0, [p_num_pts, p_num_dims])
    return (pts / np.linalg.norm(pts, axis=1)[:, np.newaxis]).astype(np.float32)


def uniform_samples_sphere(p_random_state, p_num_pts, p_num_dims):
    """Points uniform in the unit ball: surface samples scaled by u^(1/d), u uniform (pc_utils.py:144-157)."""
    surface = uniform_samples_surface_sphere(p_random_state, p_num_pts, p_num_dims)
    radius = np.power(p_random_state.uniform(0.0, 1.0, [p_num_pts, 1]), 1.0 / float(p_num_dims))
    return (surface * radius).astype(np.float32)


def poisson_disk_sampling(p_pts, p_radii):
    """Greedy Poisson-disk subset in input order (pc_utils.py:160-178): the first point is kept, and a later point is
    kept iff its distance, measured in units of ``p_radii`` per axis, to every point kept so far is at least one.
    The reference forms all n x n distances first; this keeps one row at a time (the same values, O(n) memory)."""
    kept = [0]
    for i in range(1, len(p_pts)):
        scaled = (p_pts[i][np.newaxis, :] - p_pts[kept]) / p_radii
        if np.amin(np.linalg.norm(scaled, axis=1)) >= 1.0:
            kept.append(i)
    return p_pts[kept, :]


def farthest_point_sampling(p_pts, p_num_pts, p_return_indices=False):
    """Farthest-point subset of ``p_num_pts`` points starting from point 0 (pc_utils.py:181-204): each step adds the
    point whose distance to the chosen set is largest (the first of equals)."""
    indices = [0]
    nearest = np.linalg.norm(p_pts - p_pts[0], axis=1)
    while len(indices) < p_num_pts:
        pick = np.argmax(nearest)
        indices.append(pick)
        nearest = np.minimum(nearest, np.linalg.norm(p_pts - p_pts[pick], axis=1))
    if p_return_indices:
        return p_pts[indices, :], indices
    return p_pts[indices, :]
