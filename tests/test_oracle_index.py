"""Pins the oracle's integer path (keys, sort, pillar table, neighbor lists, pooling) against the
formulations the reference's own unit tests use, brute force and invariants.  CPU only."""
import numpy as np
import pytest

from pccnn_lib_amd import synthetic


def _cloud(models, batch, num_pts, dims):
    pts = models[:batch, :num_pts, :].reshape(-1, 3)
    if dims < 3:
        pts = pts[:, :dims]
    elif dims > 3:
        pts = np.concatenate([pts[:, 0:3], pts[:, 0:dims - 3]], axis=-1)
    ids = np.repeat(np.arange(batch, dtype=np.int32), num_pts)
    return np.ascontiguousarray(pts, np.float32), ids


CASES = [(4, 1000, 0.2), (4, 100, 1.0)]


@pytest.mark.parametrize("dims", [2, 3, 6])
@pytest.mark.parametrize("batch,num_pts,radius", CASES)
def test_keys_match_unit_test_formula(oracle, models, batch, num_pts, radius, dims):
    # unit_test/test_cell_ids.py:53-65 (division by the cell size, numpy float32).
    pts, ids = _cloud(models, batch, num_pts, dims)
    cell = np.full(dims, radius, np.float32)
    mn, mx = oracle.bounding_box(pts, ids, batch)
    nc = oracle.num_cells(mn, mx, cell)
    keys = oracle.compute_keys(pts, ids, mn, nc, cell)
    cells = np.floor((pts - mn[ids]) / cell.reshape(1, -1)).astype(np.int64)
    cells = np.minimum(np.maximum(cells, 0), nc.astype(np.int64) - 1)
    expect = np.zeros(pts.shape[0], np.int64)
    accum = 1
    for i in range(dims - 1, -1, -1):
        expect += cells[:, i] * accum
        accum *= int(nc[i])
    expect += ids.astype(np.int64) * accum
    assert np.array_equal(keys, expect)


def test_keys_known_answer(oracle):
    # Hand-worked: two clouds, grid 4 x 3 x 2, cell 0.5.  Out-of-box points clamp.
    pts = np.array([[0.0, 0.0, 0.0], [0.6, 1.2, 0.9], [1.99, 1.49, 0.99], [-5.0, 9.0, 0.26],
                    [10.1, 10.1, 10.6]], np.float32)
    ids = np.array([0, 0, 0, 0, 1], np.int32)
    mn = np.array([[0, 0, 0], [10, 10, 10]], np.float32)
    nc = np.array([4, 3, 2], np.int32)
    cell = np.array([0.5, 0.5, 0.5], np.float32)
    keys = oracle.compute_keys(pts, ids, mn, nc, cell)
    # cells: (0,0,0) (1,2,1) (3,2,1) (0,2,0) | (0,0,1) in cloud 1
    assert keys.tolist() == [0, 1 * 6 + 2 * 2 + 1, 3 * 6 + 2 * 2 + 1, 2 * 2, 24 + 1]


def test_bounding_box_and_num_cells(oracle, models):
    # unit_test/test_bb.py:45-51 (np.amin / np.amax per cloud, 1e-5).
    pts, ids = _cloud(models, 4, 1000, 3)
    mn, mx = oracle.bounding_box(pts, ids, 4)
    for b in range(4):
        assert np.allclose(mn[b], pts[ids == b].min(axis=0), atol=1e-5, rtol=0)
        assert np.allclose(mx[b], pts[ids == b].max(axis=0), atol=1e-5, rtol=0)
        assert (mn[b] < pts[ids == b].min(axis=0)).all()
    nc = oracle.num_cells(mn, mx, np.full(3, 0.2, np.float32))
    assert nc.dtype == np.int32 and (nc >= 1).all()
    assert np.array_equal(nc, (((mx - mn) / np.float32(0.2)).astype(np.int32) + 1).max(axis=0))


@pytest.mark.parametrize("dims", [2, 3, 6])
@pytest.mark.parametrize("batch,num_pts,radius", CASES)
def test_grid_ds_matches_unit_test_loop(oracle, models, batch, num_pts, radius, dims):
    # unit_test/test_grid_ds.py:69-98: walk the sorted points, open/close pillar ranges.
    pts, ids = _cloud(models, batch, num_pts, dims)
    cell = np.full(dims, radius, np.float32)
    mn, mx = oracle.bounding_box(pts, ids, batch)
    nc = oracle.num_cells(mn, mx, cell)
    keys = oracle.compute_keys(pts, ids, mn, nc, cell)
    perm = oracle.argsort_keys(keys)
    assert np.array_equal(perm, np.argsort(keys, kind="stable"))
    skeys = keys[perm]
    ds = oracle.build_grid_ds(skeys, nc, batch)
    expect = np.zeros((batch, int(nc[0]), int(nc[1]), 2), np.int32)
    div = int(np.prod(nc[2:].astype(np.int64)))
    pillar = skeys // div
    for i in range(skeys.shape[0]):
        b, r = divmod(int(pillar[i]), int(nc[0]) * int(nc[1]))
        x, y = divmod(r, int(nc[1]))
        if i == 0 or pillar[i - 1] != pillar[i]:
            expect[b, x, y, 0] = i
        expect[b, x, y, 1] = i + 1
    assert np.array_equal(ds, expect)
    # invariants: non-empty ranges tile [0, N) without overlap
    flat = ds.reshape(-1, 2)
    flat = flat[flat[:, 1] > flat[:, 0]]
    flat = flat[np.argsort(flat[:, 0])]
    assert flat[0, 0] == 0 and flat[-1, 1] == skeys.shape[0]
    assert np.array_equal(flat[1:, 0], flat[:-1, 1])


def test_offsets_table(oracle):
    o3 = oracle.offsets(3)
    assert o3.shape == (9, 3) and (o3[:, 2] == 0).all()
    assert sorted(map(tuple, o3[:, :2])) == sorted((a, b) for a in (-1, 0, 1) for b in (-1, 0, 1))
    assert oracle.offsets(2).shape == (9, 2)
    o6 = oracle.offsets(6)
    assert o6.shape == (243, 6) and (o6[:, 5] == 0).all()


@pytest.mark.parametrize("dims", [2, 3, 6])
@pytest.mark.parametrize("batch,num_pts,radius", CASES)
def test_neighbors_match_brute_force(oracle, models, batch, num_pts, radius, dims):
    pts, ids = _cloud(models, batch, num_pts, dims)
    nb = oracle.neighborhood(pts, ids, pts, ids, radius)
    bf, bf_ends = oracle.brute_force_neighbors(pts, ids, pts, ids, nb["radii"])
    assert np.array_equal(nb["ends"], bf_ends)
    assert np.array_equal(oracle.canonical_pairs(nb["neighbors"]), oracle.canonical_pairs(bf))
    # unit_test/test_find_neighs.py:57-67: sqrt(sum(diff^2)) < radius in numpy float32; the op
    # multiplies by the reciprocal radius instead.  Count pairs whose decision differs.
    differ = 0
    for s in range(0, pts.shape[0], 7):
        d = pts - pts[s:s + 1]
        mask = np.logical_and(np.sqrt(np.sum(d * d, axis=-1)) < np.float32(radius), ids == ids[s])
        lo = nb["ends"][s - 1] if s > 0 else 0
        mine = set(nb["neighbors"][lo:nb["ends"][s], 0].tolist())
        differ += len(mine.symmetric_difference(np.where(mask)[0].tolist()))
    assert differ == 0
    # invariants: self is a neighbor, ends monotone, symmetric relation
    ends = nb["ends"]
    assert (np.diff(ends) >= 1).all() and ends[-1] == nb["neighbors"].shape[0]
    pairs = set(map(tuple, nb["neighbors"].tolist()))
    assert all((s, s) in pairs for s in range(0, pts.shape[0], 13))
    assert all((b, a) in pairs for a, b in list(pairs)[:2000])


def test_neighbors_samples_differ_from_points(oracle):
    rng = np.random.default_rng(5)
    pts = np.concatenate([synthetic.sphere_surface(rng, 700), synthetic.sphere_surface(rng, 500)])
    ids = np.concatenate([np.zeros(700, np.int32), np.ones(500, np.int32)])
    # samples strictly inside the points' box so that clamping never drops a neighbor
    smp = (np.concatenate([synthetic.sphere_surface(rng, 90), synthetic.sphere_surface(rng, 60)]) * 0.97)
    sids = np.concatenate([np.zeros(90, np.int32), np.ones(60, np.int32)])
    nb = oracle.neighborhood(pts, ids, smp.astype(np.float32), sids, 0.15)
    bf, bf_ends = oracle.brute_force_neighbors(smp, sids, pts, ids, nb["radii"])
    assert np.array_equal(nb["ends"], bf_ends)
    assert np.array_equal(oracle.canonical_pairs(nb["neighbors"]), oracle.canonical_pairs(bf))


@pytest.mark.parametrize("cap", [4, 9])
def test_neighbors_capped(oracle, models, cap):
    # unit_test/test_find_neighs.py:78-94: a capped sample has exactly `cap` true neighbors.
    pts, ids = _cloud(models, 4, 1000, 3)
    full = oracle.neighborhood(pts, ids, pts, ids, 0.2)
    capd = oracle.neighborhood(pts, ids, pts, ids, 0.2, max_neighbors=cap)
    fe, ce = np.diff(full["ends"], prepend=0), np.diff(capd["ends"], prepend=0)
    assert np.array_equal(ce, np.minimum(fe, cap))
    full_sets = {}
    for a, s in full["neighbors"].tolist():
        full_sets.setdefault(s, set()).add(a)
    seen = set()
    for a, s in capd["neighbors"].tolist():
        assert a in full_sets[s]
        assert (a, s) not in seen
        seen.add((a, s))


@pytest.mark.parametrize("num_pts,radius", [(1000, 0.1), (100, 3.0)])
def test_poisson_disk(oracle, models, num_pts, radius):
    # unit_test/test_pd_pooling.py:51-59 (no two selected points of a cloud closer than the radius)
    # plus maximality: every rejected point has a selected neighbor.
    pts, ids = _cloud(models, 4, num_pts, 3)
    nb = oracle.neighborhood(pts, ids, pts, ids, radius)
    spts, sids = nb["sorted_pts"], ids[nb["perm"]]
    neigh, ends = oracle.find_neighbors(spts, nb["sorted_keys"], spts, nb["sorted_keys"], nb["grid_ds"],
                                        nb["num_cells"], nb["radii"])
    sel = oracle.poisson_disk_sampling(nb["sorted_keys"], neigh, ends, nb["num_cells"]).reshape(-1)
    assert sel.shape[0] > 0
    chosen = np.zeros(spts.shape[0], bool)
    chosen[sel] = True
    for b in range(4):
        p = spts[np.logical_and(chosen, sids == b)].astype(np.float64)
        d = np.linalg.norm(p[:, None, :] - p[None, :, :], axis=-1) + np.eye(p.shape[0]) * 1e9
        assert d.min() >= radius * (1 - 1e-6)
    for s in range(spts.shape[0]):
        if not chosen[s]:
            lo = ends[s - 1] if s > 0 else 0
            assert chosen[neigh[lo:ends[s], 0]].any()


@pytest.mark.parametrize("case", ["3d", "2d", "4d"])
def test_poisson_disk_hand_worked_known_answers(oracle, case):
    # Expected ids are derived by hand from poisson_disk_sampling.cu:66-72,:82-104,:158-170 in
    # tests/golden/poisson_known_answers.py: launch (colour) order, which bit belongs to which dimension,
    # sorted order inside a cell.  A reversed colour order, the reversed bit order, both at once, or a plain
    # walk in sorted order each give another selection on these inputs.
    from tests.golden import poisson_known_answers as kat
    (keys, neigh, ends, ncells), expect = kat.CASES[case]()
    got = oracle.poisson_disk_sampling(keys, neigh, ends, ncells)
    assert got.shape == (expect.shape[0], 1)
    assert got.reshape(-1).tolist() == expect.tolist()
