"""The host-side augmentation and sampling helpers (pccnn_lib/py_utils/pc_utils.py): results and, for the random
ones, the draws they take from the caller's RandomState (a seeded script must get the same clouds)."""
import numpy as np

import pccnn_lib_amd as lib
from pccnn_lib_amd import py_utils


def _cloud(n=200, d=3, seed=0):
    return np.random.RandomState(seed).rand(n, d).astype(np.float32)


def test_names_are_exported_at_the_top_level_like_the_reference():
    for name in ("jitter_pc", "mirror_pc", "anisotropic_scale_pc", "rotate_pc_3d", "uniform_samples_surface_sphere",
                 "uniform_samples_sphere", "poisson_disk_sampling", "farthest_point_sampling"):
        assert getattr(lib, name) is getattr(py_utils, name)


def test_jitter_draws_one_gaussian_block_and_clips_it():
    pts = _cloud()
    got = py_utils.jitter_pc(np.random.RandomState(7), pts, 0.01, 0.015)
    draw = np.random.RandomState(7).randn(200, 3)
    assert np.array_equal(got, pts + np.clip(draw * 0.01, -0.015, 0.015))
    assert np.abs(got - pts).max() <= 0.015 + 1e-7 and (np.abs(got - pts) > 0.0149).any()
    unclipped = py_utils.jitter_pc(np.random.RandomState(7), pts, 0.01, 0.0)
    assert np.array_equal(unclipped, pts + draw * 0.01)
    # the state is left where one block of n x d normals leaves it
    a, b = np.random.RandomState(7), np.random.RandomState(7)
    py_utils.jitter_pc(a, pts)
    b.randn(200, 3)
    assert a.random_sample() == b.random_sample()


def test_mirror_takes_one_draw_per_axis_entry_and_flips_only_allowed_axes():
    pts, normals = _cloud(), _cloud(seed=1)
    for seed in range(6):
        draws = np.random.RandomState(seed).random_sample(3)
        allowed = [True, False, True]
        got, got_n, signs = py_utils.mirror_pc(np.random.RandomState(seed), allowed, pts, normals, True)
        expect = np.array([[-1.0 if (draws[i] > 0.5 and allowed[i]) else 1.0 for i in range(3)]], np.float32)
        assert signs.dtype == np.float32 and np.array_equal(signs, expect)
        assert np.array_equal(got, pts * expect) and np.array_equal(got_n, normals * expect)
    only_pts = py_utils.mirror_pc(np.random.RandomState(0), [True, True, True], pts)
    assert len(only_pts) == 2 and only_pts[1] is None


def test_anisotropic_scale_uses_one_factor_per_axis():
    pts = _cloud()
    got, factors = py_utils.anisotropic_scale_pc(np.random.RandomState(3), pts, 0.8, 1.3, True)
    draw = np.random.RandomState(3).random_sample((1, 3))
    assert np.array_equal(factors, draw * (1.3 - 0.8) + 0.8) and factors.shape == (1, 3)
    assert np.array_equal(got, pts * factors) and (factors >= 0.8).all() and (factors < 1.3).all()
    assert np.array_equal(py_utils.anisotropic_scale_pc(np.random.RandomState(3), pts, 0.8, 1.3), got)


def test_rotation_is_rz_ry_rx_applied_from_the_right():
    pts = _cloud()
    rotated, r = py_utils.rotate_pc_3d(np.random.RandomState(11), pts, 0.7)
    ax, ay, az = (np.random.RandomState(11).random_sample(3) - 0.5) * 2.0 * 0.7
    rx = np.array([[1, 0, 0], [0, np.cos(ax), -np.sin(ax)], [0, np.sin(ax), np.cos(ax)]])
    ry = np.array([[np.cos(ay), 0, np.sin(ay)], [0, 1, 0], [-np.sin(ay), 0, np.cos(ay)]])
    rz = np.array([[np.cos(az), -np.sin(az), 0], [np.sin(az), np.cos(az), 0], [0, 0, 1]])
    assert np.allclose(r, rz @ ry @ rx, atol=1e-15) and np.allclose(rotated, pts @ r, atol=1e-15)
    assert np.allclose(r @ r.T, np.eye(3), atol=1e-12) and abs(np.linalg.det(r) - 1.0) < 1e-12
    # a quarter turn about z alone, from the right: (1, 0, 0) -> (0, -1, 0)
    class Fixed(object):
        def random_sample(self, shape):
            return np.array([0.9, 0.1, 0.75])
    turned, rq = py_utils.rotate_pc_3d(Fixed(), np.array([[1.0, 0.0, 0.0]]), np.pi, [2])
    assert np.allclose(rq, [[0, -1, 0], [1, 0, 0], [0, 0, 1]], atol=1e-12)
    assert np.allclose(turned, [[0.0, -1.0, 0.0]], atol=1e-12)
    # disabled axes still consume their draw
    a, b = np.random.RandomState(5), np.random.RandomState(5)
    py_utils.rotate_pc_3d(a, pts, p_axes=[1])
    b.random_sample(3)
    assert a.random_sample() == b.random_sample()


def test_sphere_samples():
    surf = py_utils.uniform_samples_surface_sphere(np.random.RandomState(2), 5000, 4)
    assert surf.dtype == np.float32 and surf.shape == (5000, 4)
    assert np.allclose(np.linalg.norm(surf, axis=1), 1.0, atol=1e-6) and np.abs(surf.mean(axis=0)).max() < 0.05
    raw = np.random.RandomState(2).normal(0.0, 1.0, [5000, 4])
    assert np.array_equal(surf, (raw / np.linalg.norm(raw, axis=1)[:, None]).astype(np.float32))
    ball = py_utils.uniform_samples_sphere(np.random.RandomState(2), 20000, 3)
    radius = np.linalg.norm(ball, axis=1)
    assert ball.dtype == np.float32 and radius.max() <= 1.0 + 1e-6
    # uniform in the volume: the fraction inside radius r is r^3
    for r in (0.5, 0.8):
        assert abs((radius < r).mean() - r ** 3) < 0.02
    state = np.random.RandomState(2)
    state.normal(0.0, 1.0, [20000, 3])
    u = state.uniform(0.0, 1.0, [20000, 1])
    assert np.allclose(radius, np.power(u[:, 0], 1.0 / 3.0), atol=1e-6)


def test_poisson_disk_subset_is_the_greedy_one_in_input_order():
    pts = _cloud(400, 3, 9)
    radii = np.array([0.15, 0.2, 0.1], np.float32)
    got = py_utils.poisson_disk_sampling(pts, radii)
    # brute force over the full distance matrix, the way the reference states it
    dist = np.linalg.norm((pts[:, None, :] - pts[None, :, :]) / radii, axis=2)
    kept = [0]
    for i in range(1, 400):
        if dist[i, kept].min() >= 1.0:
            kept.append(i)
    assert np.array_equal(got, pts[kept])
    sel = dist[np.ix_(kept, kept)] + np.eye(len(kept)) * 10
    assert sel.min() >= 1.0                                         # no two kept points closer than the radii
    rest = np.setdiff1d(np.arange(400), kept)
    assert (dist[np.ix_(rest, kept)].min(axis=1) < 1.0).all()      # and every dropped point is blocked by a kept one
    # a hand-worked line: spacing 0.4, radius 1 -> points 0, 3, 6, 9
    line = np.zeros((10, 2), np.float32)
    line[:, 0] = 0.4 * np.arange(10)
    assert np.array_equal(py_utils.poisson_disk_sampling(line, np.ones(2, np.float32))[:, 0],
                          line[[0, 3, 6, 9], 0])


def test_farthest_point_sampling_starts_at_point_zero():
    line = np.array([[0.0], [1.0], [2.0], [10.0], [4.9], [5.1]])
    got, idx = py_utils.farthest_point_sampling(line, 4, True)
    # 0 -> farthest 10 (index 3) -> farthest from {0, 10}: 5.1 is 4.9 away, 4.9 is 4.9 away: the first of equals
    assert [int(i) for i in idx] == [0, 3, 4, 2] and np.array_equal(got, line[[0, 3, 4, 2]])
    pts = _cloud(300, 3, 4)
    sub, idx = py_utils.farthest_point_sampling(pts, 20, True)
    assert len(set(int(i) for i in idx)) == 20 and np.array_equal(sub, pts[idx])
    assert np.array_equal(py_utils.farthest_point_sampling(pts, 20), sub)
    # each pick is the point farthest from the picks before it
    for step in range(1, 20):
        d = np.min(np.linalg.norm(pts[:, None, :] - pts[idx[:step]][None, :, :], axis=2), axis=1)
        assert d[idx[step]] == d.max()
