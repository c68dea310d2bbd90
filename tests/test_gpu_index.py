"""HIP path vs the CPU oracle for the integer part of the path: bit-exact keys, permutation, pillar
table and neighbor lists (compared after sorting pairs by (sample, neighbor id)), Poisson-disk selection."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, t

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _cloud(models, batch, num_pts):
    pts = np.ascontiguousarray(models[:batch, :num_pts, :].reshape(-1, 3), np.float32)
    return pts, np.repeat(np.arange(batch, dtype=np.int32), num_pts)


def _compare_neighborhoods(oracle, got, exp):
    for key in ("aabb_min", "aabb_max", "num_cells", "keys", "perm", "sorted_keys", "sorted_pts", "grid_ds",
                "sample_keys", "ends"):
        assert np.array_equal(got[key], exp[key]), key
    assert np.array_equal(oracle.canonical_pairs(got["neigh_sorted"]), oracle.canonical_pairs(exp["neigh_sorted"]))
    assert np.array_equal(oracle.canonical_pairs(got["neighbors"]), oracle.canonical_pairs(exp["neighbors"]))
    # this build's own order: ascending sorted-point index inside each sample, same as the oracle's
    assert np.array_equal(got["neigh_sorted"], exp["neigh_sorted"])


@pytest.mark.parametrize("batch,num_pts,radius", [(4, 1000, 0.2), (4, 100, 1.0), (2, 1024, 0.05), (1, 37, 0.3)])
@pytest.mark.parametrize("use_order,use_table", [(True, False), (False, False), (True, True), (False, True)])
def test_reference_clouds_bit_exact(ops, oracle, models, batch, num_pts, radius, use_order, use_table):
    # every combination of the two search accelerators (key-ordered queries, per-cell start table)
    pts, ids = _cloud(models, batch, num_pts)
    exp = oracle.neighborhood(pts, ids, pts, ids, radius)
    got = gpu_neighborhood(ops, pts, ids, pts, ids, radius, batch, use_order=use_order, use_table=use_table)
    _compare_neighborhoods(oracle, got, exp)


def test_config1_sphere_clouds(ops, oracle):
    # 2 x 1024 points on the unit sphere, cell = radius = 0.1
    pts = np.concatenate([synthetic.sphere_surface(np.random.default_rng(s), 1024) for s in (0, 1)])
    ids = np.repeat(np.arange(2, dtype=np.int32), 1024)
    exp = oracle.neighborhood(pts, ids, pts, ids, 0.1)
    got = gpu_neighborhood(ops, pts, ids, pts, ids, 0.1, 2)
    _compare_neighborhoods(oracle, got, exp)
    bf, bf_ends = oracle.brute_force_neighbors(pts, ids, pts, ids, exp["radii"])
    assert np.array_equal(got["ends"], bf_ends)
    assert np.array_equal(oracle.canonical_pairs(got["neighbors"]), oracle.canonical_pairs(bf))


def test_primitive_clouds_medium(ops, oracle):
    pts, ids = synthetic.primitives(3, 4, 4096)
    exp = oracle.neighborhood(pts, ids, pts, ids, 0.05)
    got = gpu_neighborhood(ops, pts, ids, pts, ids, 0.05, 4)
    _compare_neighborhoods(oracle, got, exp)


def test_samples_differ_from_points(ops, oracle):
    pts, ids = synthetic.primitives(5, 3, 2000)
    rng = np.random.default_rng(1)
    pick = np.sort(rng.choice(pts.shape[0], 700, replace=False))
    smp = (pts[pick] + rng.normal(0, 0.004, (700, 3))).astype(np.float32)   # some fall outside the box: clamped
    sids = ids[pick]
    exp = oracle.neighborhood(pts, ids, smp, sids, 0.08)
    for use_table in (False, True):
        got = gpu_neighborhood(ops, pts, ids, smp, sids, 0.08, 3, use_table=use_table)
        _compare_neighborhoods(oracle, got, exp)


@pytest.mark.parametrize("num_samples", [1400, 330, 40])
def test_few_samples_against_many_points(ops, oracle, num_samples):
    # A pooling level: far fewer samples than points.  Below a quarter, and again below a sixteenth, of the point
    # count several lanes share one sample; the lists (and the capped subsets, which depend on the walk order) must be
    # those of the one-lane walk and of the oracle, pair for pair.
    pts, ids = synthetic.primitives(9, 3, 2400)
    rng = np.random.default_rng(num_samples)
    pick = np.sort(rng.choice(pts.shape[0], num_samples, replace=False))
    smp = (pts[pick] + rng.normal(0, 0.004, (num_samples, 3))).astype(np.float32)
    sids = ids[pick]
    for cap in (0, 9):
        exp = oracle.neighborhood(pts, ids, smp, sids, 0.12, max_neighbors=cap)
        for use_order, use_table in ((True, True), (False, False)):
            got = gpu_neighborhood(ops, pts, ids, smp, sids, 0.12, 3, max_neighbors=cap, use_order=use_order,
                                   use_table=use_table)
            assert np.array_equal(got["ends"], exp["ends"])
            assert np.array_equal(got["neigh_sorted"], exp["neigh_sorted"])
            assert np.array_equal(got["neighbors"], exp["neighbors"])
    assert np.diff(exp["ends"], prepend=0).max() == 9      # the cap binds


@pytest.mark.parametrize("cap", [4, 16])
def test_capped_neighbors(ops, oracle, models, cap):
    pts, ids = _cloud(models, 4, 1000)
    exp = oracle.neighborhood(pts, ids, pts, ids, 0.2, max_neighbors=cap)
    got = gpu_neighborhood(ops, pts, ids, pts, ids, 0.2, 4, max_neighbors=cap)
    assert np.array_equal(got["ends"], exp["ends"])
    assert np.diff(got["ends"], prepend=0).max() == cap
    # same deterministic even-spaced subset as the oracle's restatement
    assert np.array_equal(got["neigh_sorted"], exp["neigh_sorted"])


def test_presorted_samples_give_the_same_lists(ops):
    # samples handed over in key order (as sort_keys leaves them) against the same samples gathered through
    # sample_order: identical pair lists, for samples that are the points and for a distinct sample set, capped or not
    pts, ids = synthetic.primitives(31, 3, 2000)
    rng = np.random.default_rng(31)
    pick = np.sort(rng.choice(pts.shape[0], 1500, replace=False))
    for smp, sids in ((pts, ids), (pts[pick] + np.float32(0.003), ids[pick])):
        for cap in (0, 7):
            g = gpu_neighborhood(ops, pts, ids, smp, sids, 0.08, 3, max_neighbors=cap)
            d = g["dev"]
            ts, tsi = t(smp), t(sids)
            skey = ops.compute_keys(ts, tsi, t(g["aabb_min"]), d["nc"], d["radii"])
            bits = ops.key_bits_for(d["nc"].tolist(), 3)
            sk, order, sp = ops.sort_keys(skey, bits, ts)
            neigh, ends = ops.find_neighbors_ex(d["spts"], d["skeys"], sp, sk, d["ds"], d["nc"], d["radii"], cap, order,
                                                d["perm"], samples_presorted=True)
            assert np.array_equal(neigh.cpu().numpy(), g["neighbors"]) and np.array_equal(ends.cpu().numpy(), g["ends"])


def test_degenerate_inputs(ops, oracle):
    # all points in one cell; a single point; duplicate points
    pts = np.tile(np.array([[0.5, 0.5, 0.5]], np.float32), (130, 1))
    pts[:65] += np.random.default_rng(0).normal(0, 1e-3, (65, 3)).astype(np.float32)
    ids = np.zeros(130, np.int32)
    exp = oracle.neighborhood(pts, ids, pts, ids, 0.5)
    got = gpu_neighborhood(ops, pts, ids, pts, ids, 0.5, 1)
    _compare_neighborhoods(oracle, got, exp)
    assert got["ends"][-1] == 130 * 130
    one = np.array([[1.0, 2.0, 3.0]], np.float32)
    got = gpu_neighborhood(ops, one, np.zeros(1, np.int32), one, np.zeros(1, np.int32), 0.1, 1)
    assert got["neighbors"].tolist() == [[0, 0]] and got["ends"].tolist() == [1]


def test_empty_sample_set(ops):
    pts, ids = synthetic.primitives(1, 1, 256)
    g = gpu_neighborhood(ops, pts, ids, pts, ids, 0.1, 1)["dev"]
    neigh, ends = ops.find_neighbors_ex(g["spts"], g["skeys"], torch.empty((0, 3), device=DEV),
                                        torch.empty((0,), dtype=torch.int64, device=DEV), g["ds"], g["nc"],
                                        g["radii"], 0)
    assert tuple(neigh.shape) == (0, 2) and tuple(ends.shape) == (0,)


def test_sort_is_stable_and_handles_many_passes(ops):
    rng = np.random.default_rng(7)
    # digit widths 8 to 11 and 1 to 6 passes: up to 2^18 keys take digits of up to 11 bits, more keys of up to 9
    for n, bits in ((1, 8), (2049, 3), (100000, 20), (70001, 40), (5000, 63), (1000, 9), (4000, 11), (60000, 18),
                    (60000, 22), (300000, 18), (300000, 26), (300000, 5)):
        keys = rng.integers(0, 2 ** min(bits, 62), n, dtype=np.int64)
        pts = rng.normal(size=(n, 3)).astype(np.float32)
        skeys, perm, spts = ops.sort_keys(t(keys), bits, t(pts))
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(perm.cpu().numpy(), order.astype(np.int32)), (n, bits)
        assert np.array_equal(skeys.cpu().numpy(), keys[order])
        assert np.array_equal(spts.cpu().numpy(), pts[order])


def test_poisson_disk_matches_oracle(ops, oracle, models):
    for num_pts, radius in ((1000, 0.1), (100, 3.0)):
        pts, ids = _cloud(models, 4, num_pts)
        exp = oracle.neighborhood(pts, ids, pts, ids, radius)
        e_neigh, e_ends = oracle.find_neighbors(exp["sorted_pts"], exp["sorted_keys"], exp["sorted_pts"],
                                                exp["sorted_keys"], exp["grid_ds"], exp["num_cells"], exp["radii"])
        e_sel = oracle.poisson_disk_sampling(exp["sorted_keys"], e_neigh, e_ends, exp["num_cells"])
        g = gpu_neighborhood(ops, pts, ids, pts, ids, radius, 4)["dev"]
        neigh, ends = ops.find_neighbors_ex(g["spts"], g["skeys"], g["spts"], g["skeys"], g["ds"], g["nc"],
                                            g["radii"], 0)
        sel = ops.poisson_disk_sampling(g["skeys"], neigh, ends, g["nc"])
        assert sel.dtype == torch.int64 and sel.shape[1] == 1
        assert np.array_equal(sel.cpu().numpy(), e_sel)


@pytest.mark.parametrize("case", ["3d", "2d", "4d"])
def test_poisson_disk_hand_worked_known_answers(ops, case):
    # the same hand-derived selections that pin the oracle (tests/golden/poisson_known_answers.py), asked of the
    # HIP path directly: colour order, bit <-> dimension, sorted order inside a cell
    from tests.golden import poisson_known_answers as kat
    (keys, neigh, ends, ncells), expect = kat.CASES[case]()
    sel = ops.poisson_disk_sampling(t(keys), t(neigh), t(ends), t(ncells))
    assert sel.dtype == torch.int64 and tuple(sel.shape) == (expect.shape[0], 1)
    assert sel.cpu().numpy().reshape(-1).tolist() == expect.tolist()


@pytest.mark.parametrize("batch,num_pts,radius,use_table", [(4, 1000, 0.1, True), (3, 4000, 0.05, False),
                                                            (1, 3000, 0.45, True), (2, 2500, 0.3, False),
                                                            (1, 40, 5.0, True)])
def test_poisson_disk_from_the_grid_equals_the_list_version(ops, oracle, batch, num_pts, radius, use_table):
    # The list-free selection (flags of the walk's index ranges, positions only of flagged candidates) must pick
    # exactly the points the neighbor-list version and the oracle pick; the large radii put hundreds of points in a
    # cell, so a cell takes several rounds of 64.
    pts, ids = synthetic.primitives(70 + batch, batch, num_pts)
    exp = oracle.neighborhood(pts, ids, pts, ids, radius)
    e_neigh, e_ends = oracle.find_neighbors(exp["sorted_pts"], exp["sorted_keys"], exp["sorted_pts"],
                                            exp["sorted_keys"], exp["grid_ds"], exp["num_cells"], exp["radii"])
    e_sel = oracle.poisson_disk_sampling(exp["sorted_keys"], e_neigh, e_ends, exp["num_cells"])
    g = gpu_neighborhood(ops, pts, ids, pts, ids, radius, batch)["dev"]
    table = ops.build_cell_table(g["skeys"], batch * int(np.prod(g["nc"].tolist()))) if use_table else None
    sel = ops.poisson_disk_sampling_grid(g["spts"], g["skeys"], g["ds"], g["nc"], g["radii"], cell_table=table)
    assert sel.dtype == torch.int64 and sel.shape[1] == 1
    assert np.array_equal(sel.cpu().numpy(), e_sel)
    neigh, ends = ops.find_neighbors_ex(g["spts"], g["skeys"], g["spts"], g["skeys"], g["ds"], g["nc"], g["radii"], 0)
    assert torch.equal(sel, ops.poisson_disk_sampling(g["skeys"], neigh, ends, g["nc"]))


def test_num_cells_matches_the_reference_arithmetic(ops, oracle):
    # Grid.py:26-28: fp32 division, truncation towards zero, + 1, maximum over the clouds
    rng = np.random.default_rng(12)
    for dims in (2, 3, 6):
        mn = rng.uniform(-2, 0, (5, dims)).astype(np.float32)
        mx = (mn + rng.uniform(0.01, 3, (5, dims))).astype(np.float32)
        for cell in (0.05, 0.1, 0.37):
            cs = np.full(dims, cell, np.float32)
            got = ops.num_cells(t(mn), t(mx), t(cs)).cpu().numpy()
            assert np.array_equal(got, oracle.num_cells(mn, mx, cs))
            assert np.array_equal(got, (((mx - mn) / cs).astype(np.int32) + 1).max(axis=0))


def test_run_twice_is_bitwise_identical(ops):
    pts, ids = synthetic.primitives(11, 2, 3000)
    a = gpu_neighborhood(ops, pts, ids, pts, ids, 0.06, 2)
    b = gpu_neighborhood(ops, pts, ids, pts, ids, 0.06, 2)
    assert np.array_equal(a["neighbors"], b["neighbors"]) and np.array_equal(a["ends"], b["ends"])


def test_drop_in_find_neighbors_and_object_api_agree(ops, oracle):
    # the reference-signature op (sorts the queries and builds the cell table by itself above 4096 samples)
    # and the Pointcloud / Grid / Neighborhood objects give the oracle's lists
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(21, 3, 2500)
    exp = oracle.neighborhood(pts, ids, pts, ids, 0.07)
    g = gpu_neighborhood(ops, pts, ids, pts, ids, 0.07, 3)
    d = g["dev"]
    neigh, ends = ops.find_neighbors(d["spts"], d["skeys"], d["samples"], t(g["sample_keys"]), d["ds"], d["nc"],
                                     d["radii"], 0)
    assert np.array_equal(neigh.cpu().numpy(), exp["neigh_sorted"]) and np.array_equal(ends.cpu().numpy(), exp["ends"])
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, torch.full((3,), 0.07, device=DEV), 0)
    assert nbh.grid_.cell_table_ is not None
    assert np.array_equal(nbh.neighbors_.cpu().numpy(), exp["neighbors"])
    assert np.array_equal(nbh.start_ids_.cpu().numpy(), exp["ends"])
    assert np.array_equal(nbh.grid_.cell_ids_.cpu().numpy(), exp["keys"])
    assert np.array_equal(nbh.grid_.sorted_ids_.cpu().numpy(), exp["perm"].astype(np.int64))
    assert np.array_equal(nbh.grid_.grid_ds_.cpu().numpy(), exp["grid_ds"])


@pytest.mark.parametrize("num_pts", [100000, 200000])
def test_scene_scale_properties(ops, num_pts):
    # A room (the generator of the million-point configuration) checked through size-independent properties: sorted
    # keys, permutation, self-membership, symmetry, monotone ends.  100 000 samples run 4 lanes per sample,
    # 200 000 the one-lane walk.
    pts = synthetic.room(4, num_pts)
    ids = np.zeros(pts.shape[0], np.int32)
    g = gpu_neighborhood(ops, pts, ids, pts, ids, 0.05, 1, use_table=True)
    g2 = gpu_neighborhood(ops, pts, ids, pts, ids, 0.05, 1, use_table=False, use_order=False)
    assert np.array_equal(g["neighbors"], g2["neighbors"]) and np.array_equal(g["ends"], g2["ends"])
    assert np.all(np.diff(g["sorted_keys"]) >= 0)
    assert np.array_equal(np.sort(g["perm"]), np.arange(pts.shape[0]))
    ends, neigh = g["ends"], g["neighbors"]
    assert ends[-1] == neigh.shape[0] and np.all(np.diff(ends, prepend=0) >= 1)
    assert np.array_equal(neigh[:, 1], np.repeat(np.arange(pts.shape[0]), np.diff(ends, prepend=0)))
    d = np.linalg.norm(pts[neigh[:, 0]].astype(np.float64) - pts[neigh[:, 1]].astype(np.float64), axis=1)
    assert d.max() < 0.05 * (1 + 1e-5)
    fwd = neigh[:, 0].astype(np.int64) * pts.shape[0] + neigh[:, 1]
    bwd = neigh[:, 1].astype(np.int64) * pts.shape[0] + neigh[:, 0]
    assert np.array_equal(np.sort(fwd), np.sort(bwd))
    assert np.count_nonzero(neigh[:, 0] == neigh[:, 1]) == pts.shape[0]
    # and complete: the pair count of a few hundred samples equals a float64 count over all points, boundary cases
    # (within 1e-6 of the radius, where fp32 and float64 may disagree) set aside
    for s_i in np.random.default_rng(1).choice(pts.shape[0], 300, replace=False):
        dist = np.linalg.norm(pts.astype(np.float64) - pts[s_i].astype(np.float64), axis=1)
        sure, maybe = np.count_nonzero(dist < 0.05 * (1 - 1e-6)), np.count_nonzero(dist < 0.05 * (1 + 1e-6))
        count = ends[s_i] - (ends[s_i - 1] if s_i > 0 else 0)
        assert sure <= count <= maybe, s_i


def test_one_lane_walk_with_more_candidates_than_its_masks_hold(ops):
    # 140 000 samples run the one-lane walk, whose count pass records 1024 candidate slots per sample for the fill
    # pass; 1500 points inside a 4 mm cube give their samples more than that, so the fill pass tests the rest itself.
    # Every list of the clump and of 200 other samples against a float64 count over all points (boundary cases
    # within 1e-6 of the radius set aside), plus the properties that hold for the whole list.
    rng = np.random.default_rng(11)
    clump = (np.float32(0.5) + np.float32(0.004) * rng.random((1500, 3), dtype=np.float32)).astype(np.float32)
    pts = np.concatenate([synthetic.room(6, 138500), clump])
    pts = pts[rng.permutation(pts.shape[0])]
    ids = np.zeros(pts.shape[0], np.int32)
    g = gpu_neighborhood(ops, pts, ids, pts, ids, 0.05, 1, use_table=True)
    ends, neigh = g["ends"], g["neighbors"]
    counts = np.diff(ends, prepend=0)
    assert ends[-1] == neigh.shape[0] and counts.max() >= 1500
    assert np.array_equal(neigh[:, 1], np.repeat(np.arange(pts.shape[0]), counts))
    fwd = neigh[:, 0].astype(np.int64) * pts.shape[0] + neigh[:, 1]
    bwd = neigh[:, 1].astype(np.int64) * pts.shape[0] + neigh[:, 0]
    assert np.array_equal(np.sort(fwd), np.sort(bwd))
    in_clump = np.flatnonzero(np.all(np.abs(pts - np.float32(0.502)) < 0.0021, axis=1))
    assert in_clump.size >= 1500
    p64 = pts.astype(np.float64)
    for s_i in np.concatenate([in_clump[:60], rng.choice(pts.shape[0], 200, replace=False)]):
        dist = np.linalg.norm(p64 - p64[s_i], axis=1)
        sure, maybe = dist < 0.05 * (1 - 1e-6), dist < 0.05 * (1 + 1e-6)
        mine = neigh[(ends[s_i] - counts[s_i]):ends[s_i], 0]
        assert np.count_nonzero(sure) <= mine.size <= np.count_nonzero(maybe), s_i
        assert np.all(maybe[mine]) and np.all(np.isin(np.flatnonzero(sure), mine)), s_i


def test_row_gather_and_permutation_inverse(ops):
    # what the reference's Python does with torch.index_select: rows of 1, 3, 8 and 33 floats (16-byte and 4-byte
    # paths), an index with repeats, and the inverse of a permutation
    rng = np.random.default_rng(2)
    for width in (None, 3, 8, 33):
        src = rng.normal(size=(5000,) if width is None else (5000, width)).astype(np.float32)
        index = rng.integers(0, 5000, 7001).astype(np.int32)
        got = ops.gather_rows(t(src), t(index)).cpu().numpy()
        assert np.array_equal(got, src[index])
    perm = rng.permutation(100001).astype(np.int32)
    inverse = ops.invert_permutation(t(perm)).cpu().numpy()
    assert np.array_equal(inverse[perm], np.arange(100001))
    assert ops.gather_rows(t(np.zeros((4, 8), np.float32)), t(np.zeros(0, np.int32))).shape == (0, 8)


def test_pair_count_beyond_32_bits_is_an_error(ops):
    # 50 000 points inside one search radius are 2.5e9 pairs: the offsets are 32-bit as in the reference, so the
    # search refuses instead of returning wrapped offsets
    import pccnn_lib_amd as lib
    n = 50000
    pts = t(np.random.default_rng(3).random((n, 3), dtype=np.float32) * 0.1)
    pc = lib.pc.Pointcloud(pts, torch.zeros(n, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="pairs"):
        lib.pc.layers.conv_base.build_neighborhood(pc, pc, torch.full((3,), 1.0, device=DEV), 0)
    # 70 000 such points are 4.9e9 pairs: the 32-bit running total wraps past 2^32 to a positive number
    # (about 6e8), which only the 64-bit total that the count pass leaves in its workspace gives away
    n = 70000
    pts = t(np.random.default_rng(4).random((n, 3), dtype=np.float32) * 0.1)
    pc = lib.pc.Pointcloud(pts, torch.zeros(n, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="pairs"):
        lib.pc.layers.conv_base.build_neighborhood(pc, pc, torch.full((3,), 1.0, device=DEV), 0)


def test_grid_ops_on_an_empty_cloud(ops):
    # no points: the grid-based selection and density return empty results without launching anything
    pts, ids = synthetic.primitives(1, 1, 256)
    g = gpu_neighborhood(ops, pts, ids, pts, ids, 0.1, 1)["dev"]
    none_pts = torch.empty((0, 3), device=DEV)
    none_keys = torch.empty((0,), dtype=torch.int64, device=DEV)
    sel = ops.poisson_disk_sampling_grid(none_pts, none_keys, g["ds"], g["nc"], g["radii"])
    assert tuple(sel.shape) == (0, 1) and sel.dtype == torch.int64
    pdf, normed = ops.compute_pdf_grid(3, g["radii"] * 0.25, none_pts, none_keys, None, g["ds"], g["nc"], g["radii"], 300,
                                       with_normalized=True)
    assert tuple(pdf.shape) == (0,) and tuple(normed.shape) == (0,)
    with pytest.raises(RuntimeError):
        ops.compute_pdf_grid(3, g["radii"][:2].contiguous(), g["spts"], g["skeys"], None, g["ds"], g["nc"], g["radii"])


def test_bounding_box_is_remembered_until_the_cloud_changes(ops):
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(5, 2, 500)
    pc = lib.pc.Pointcloud(t(pts), t(ids))
    first = lib.pc.BoundingBox(pc)
    again = lib.pc.BoundingBox(pc)
    assert again.min_ is first.min_ and again.max_ is first.max_          # same cloud, untouched: not recomputed
    pc.pts_.mul_(2.0)                                                     # written in place: computed again
    scaled = lib.pc.BoundingBox(pc)
    assert scaled.min_ is not first.min_
    assert torch.allclose(scaled.max_ - scaled.min_, 2.0 * (first.max_ - first.min_), atol=1e-5)
    pc.pts_ = pc.pts_ + 1.0                                               # replaced: computed again
    moved = lib.pc.BoundingBox(pc)
    assert torch.allclose(moved.min_, scaled.min_ + 1.0, atol=1e-5)


@pytest.mark.parametrize("num_pts", [40000, 200000])
def test_capped_lists_are_the_ruled_subset_of_the_full_lists(ops, num_pts):
    # With a cap, sample by sample, hit number r of raw (in walk order) is kept iff floor((r + 1) cap / raw) >
    # floor(r cap / raw).  Checked against the uncapped search of the same grid, restated with numpy, at a size that
    # runs 8 lanes per sample (40 000) and at one that runs the one-lane walk (200 000).
    import pccnn_lib_amd as lib
    cap = 6
    pts = t(synthetic.room(8, num_pts))
    pc = lib.pc.Pointcloud(pts, torch.zeros(num_pts, dtype=torch.int32, device=DEV))
    radii = torch.full((3,), 0.12 if num_pts < 100000 else 0.06, device=DEV)
    full = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    capped = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, cap)
    f_neigh, f_ends = full.neighbors_.cpu().numpy(), full.start_ids_.cpu().numpy().astype(np.int64)
    c_neigh, c_ends = capped.neighbors_.cpu().numpy(), capped.start_ids_.cpu().numpy().astype(np.int64)
    raw = np.diff(f_ends, prepend=0)
    assert raw.max() > 4 * cap                                     # the cap bites
    assert np.array_equal(np.diff(c_ends, prepend=0), np.minimum(raw, cap))
    starts = f_ends - raw
    rank = np.arange(f_neigh.shape[0], dtype=np.int64) - np.repeat(starts, raw)
    raw_of_pair = np.repeat(raw, raw)
    keep = (raw_of_pair <= cap) | (((rank + 1) * cap) // raw_of_pair > (rank * cap) // raw_of_pair)
    assert np.array_equal(c_neigh, f_neigh[keep])


@pytest.mark.parametrize("batch,num_pts,radius", [(3, 2500, 0.08), (1, 6000, 0.05)])
def test_cell_average_pooling(ops, oracle, batch, num_pts, radius):
    # pccnn_lib/pc/PointPooling.py:71-83 (one group per occupied cell: np.unique of the cell keys) and :97-102
    # (scatter_mean / scatter_max over the groups)
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(31, batch, num_pts)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pool = lib.pc.PointPooling(pc, torch.full((3,), radius, device=DEV), "cell_average")
    exp = oracle.neighborhood(pts, ids, pts, ids, radius)
    uniq, inverse = np.unique(exp["keys"], return_inverse=True)
    assert pool.num_pooling_pts_ == uniq.shape[0] and pool.pooling_ids_.dtype == torch.int64
    assert np.array_equal(pool.pooling_ids_.cpu().numpy(), inverse.reshape(-1))
    rng = np.random.default_rng(31)
    vals = rng.normal(size=(pts.shape[0], 5)).astype(np.float32)
    sums = np.zeros((uniq.shape[0], 5), np.float64)
    np.add.at(sums, inverse.reshape(-1), vals.astype(np.float64))
    counts = np.bincount(inverse.reshape(-1), minlength=uniq.shape[0]).astype(np.float64)
    maxes = np.full((uniq.shape[0], 5), -np.inf, np.float32)
    np.maximum.at(maxes, inverse.reshape(-1), vals)
    mean = pool.pool_tensor(t(vals))
    assert tuple(mean.shape) == (uniq.shape[0], 5)
    assert np.abs(mean.cpu().numpy() - sums / counts[:, None]).max() < 1e-5
    assert np.array_equal(pool.pool_tensor(t(vals), max_pool=True).cpu().numpy(), maxes)


def test_grid_size_on_the_host_equals_the_device_result(ops):
    # a cell size given as host values: Grid.num_cells_host() redoes the fp32 arithmetic of Grid.py:26-28 in numpy on
    # the box's host copy instead of reading the device result back; both must agree for every cloud and cell size
    import pccnn_lib_amd as lib
    rng = np.random.default_rng(77)
    for trial in range(40):
        batch = int(rng.integers(1, 5))
        pts, ids = synthetic.primitives(100 + trial, batch, 700)
        pts = (pts * rng.uniform(0.3, 7.0, (1, 3))).astype(np.float32)
        pc = lib.pc.Pointcloud(pts, ids, device=DEV)
        for cell in (float(rng.uniform(0.01, 0.5)), rng.uniform(0.01, 0.5, 3).astype(np.float32), 0.05, 0.1, 0.25):
            grid = lib.pc.Grid(pc, lib.pc.BoundingBox(pc), cell)
            assert grid.num_cells_host() == grid.num_cells_.tolist()
    # a cloud made from pooled batch ids knows its number of clouds without reading the ids back
    pts, ids = synthetic.primitives(5, 3, 2000)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pool = lib.pc.PointPooling(pc, 0.1)
    out = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
    assert out.batch_size_host_ == 3 and int(out.batch_size_) == 3 and int(torch.max(out.batch_ids_)) == 2


@pytest.mark.parametrize("batch,num_pts,radius", [(3, 3000, 0.08), (1, 500, 0.3), (4, 20000, 0.04)])
def test_one_call_pooling_density_and_neighborhood_equal_the_step_by_step_routes(ops, monkeypatch, batch, num_pts, radius):
    # PointPooling, Pointcloud.compute_pdf and Neighborhood run their chain of launches as one native call when the grid size is known on
    # the host; the same launches step by step (the route of every other case) must give the same tensors
    import pccnn_lib_amd as lib
    from pccnn_lib_amd.pc import neighborhood, point_cloud, point_pooling
    pts, ids = synthetic.primitives(31 + batch, batch, num_pts)

    def run(one_call):
        monkeypatch.setattr(point_pooling, "ONE_CALL", one_call)
        monkeypatch.setattr(neighborhood, "ONE_CALL", one_call)
        monkeypatch.setattr(point_cloud, "ONE_CALL", one_call)
        pc = lib.pc.Pointcloud(pts, ids, device=DEV)
        pool = lib.pc.PointPooling(pc, radius)
        out_pc = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
        pc.compute_pdf(0.25 * radius)
        # the pooled cloud's box: computed on request (step by step), or come back with the selection (one call)
        assert (getattr(out_pc, "aabb_cache_", None) is not None) == one_call
        box = lib.pc.BoundingBox(out_pc)
        fresh_min, fresh_max = ops.bounding_box(out_pc.pts_, out_pc.batch_ids_, batch)
        assert torch.equal(box.min_, fresh_min) and torch.equal(box.max_, fresh_max)
        assert np.array_equal(box.host()[0], fresh_min.cpu().numpy()) and np.array_equal(box.host()[1], fresh_max.cpu().numpy())
        got = [pool.pooling_ids_, pc.pts_unnorm_pdf_, pc.pts_pdf_, box.min_, box.max_, out_pc.pts_, out_pc.batch_ids_,
               pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_)]       # (a second request: gathered anew)
        assert torch.equal(got[-2], pc.pts_[pool.pooling_ids_]) and got[-2] is not out_pc.pts_
        for samples, cap, key_order in ((out_pc, 0, False), (pc, 0, False), (out_pc, 5, False), (out_pc, 0, True)):
            grid = lib.pc.Grid(pc, lib.pc.BoundingBox(pc), 2.0 * radius)
            if not one_call:
                grid.compute_cell_ids()
                grid.build_ds()
            nbh = lib.pc.Neighborhood(grid, samples, cap, key_order)
            got += [nbh.neighbors_key_order_ if key_order else nbh.neighbors_original_, nbh.neighbors_,
                    nbh.start_ids_, grid.num_cells_, grid.cell_ids_, grid.sorted_cell_ids_, grid.sorted_ids_,
                    grid.sorted_pts_, grid.grid_ds_, grid.cell_table_]
        return got

    a, b = run(False), run(True)
    assert len(a) == len(b) and a[0].dtype == torch.int64 and a[0].shape[0] > 0
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and tuple(x.shape) == tuple(y.shape) and torch.equal(x, y)


@pytest.mark.parametrize("num_pts", [900, 30000])
def test_pooling_settles_on_first_use_with_other_work_queued_in_between(ops, monkeypatch, num_pts):
    # the one-call pooling queues its work and waits for the selection's size only when a result is asked for;
    # density, allocations of every size and a second pooling queued in between change nothing, and the result is
    # that of the pooling that waits in its constructor
    import pccnn_lib_amd as lib
    from pccnn_lib_amd.pc.point_pooling import PointPooling
    pts, ids = synthetic.primitives(57, 3, num_pts)
    radius = 0.06

    def run(later):
        monkeypatch.setattr(PointPooling, "LATER", later)
        pc = lib.pc.Pointcloud(pts, ids, device=DEV)
        pool = PointPooling(pc, radius)
        assert (pool.pending_ is not None) == later
        other = PointPooling(pc, 2.0 * radius)
        unused = PointPooling(pc, 3.0 * radius)
        del unused                                  # never asked for: waits for its queued copy, then lets go
        pc.compute_pdf(0.25 * radius)
        junk = [torch.full((size,), 7, dtype=torch.int32, device=DEV) for size in (64, 5000, 3 * num_pts, 400000)]
        out_pts, out_ids = pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_)
        assert pool.pending_ is None and all(int(j[0]) == 7 for j in junk)
        box = out_pts.pccnn_pooled_box_.box
        return [pool.pooling_ids_, out_pts, out_ids, box[0], box[1], torch.as_tensor(box[2][0]),
                torch.as_tensor(box[2][1]), other.pooling_ids_, pc.pts_unnorm_pdf_]

    a, b = run(False), run(True)
    assert a[0].shape[0] > 0 and torch.equal(a[1], t(pts)[a[0]])
    mn, mx = ops.bounding_box(a[1], a[2], 3)
    assert torch.equal(a[3], mn) and torch.equal(a[4], mx) and torch.equal(a[5], mn.cpu()) and torch.equal(a[6], mx.cpu())
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and tuple(x.shape) == tuple(y.shape) and torch.equal(x, y)


@pytest.mark.parametrize("m", [4096, 4097, 8193, 16385, 32768, 32769, 49152, 49153, 70000])
def test_start_ids_are_the_running_sum_of_the_counts_at_every_scan_size(ops, m):
    # the scan behind start_ids_ runs as one workgroup with 4, 8, 16, 32 or 48 elements per thread, or as three
    # launches: sample counts on either side of every limit, start_ids_ against numpy's cumulative sum of the
    # per-sample pair counts
    rng = np.random.default_rng(m)
    pts = rng.random((20000, 3), dtype=np.float32)
    samples = rng.random((m, 3), dtype=np.float32)
    nb = gpu_neighborhood(ops, pts, np.zeros(20000, np.int32), samples, np.zeros(m, np.int32), 0.03, 1)
    counts = np.bincount(nb["neighbors"][:, 1], minlength=m)
    assert nb["ends"].shape == (m,) and nb["neighbors"].shape[0] > m
    assert np.array_equal(nb["ends"], np.cumsum(counts))


def test_bounding_box_comes_back_on_the_host_with_the_same_call(ops):
    pts, ids = synthetic.primitives(3, 5, 800)
    mn, mx, (host_mn, host_mx) = ops.bounding_box_host(t(pts), t(ids), 5)
    mn2, mx2 = ops.bounding_box(t(pts), t(ids), 5)
    assert torch.equal(mn, mn2) and torch.equal(mx, mx2)
    assert np.array_equal(host_mn, mn.cpu().numpy()) and np.array_equal(host_mx, mx.cpu().numpy())
    assert host_mn.dtype == np.float32 and host_mn.shape == (5, 3)


@pytest.mark.parametrize("num_pts,batch", [(1000, 7), (16384, 64), (16385, 3), (40000, 70)])
def test_bounding_box_with_interleaved_clouds_and_an_empty_one(ops, num_pts, batch):
    # the one-workgroup kernel of small inputs and the chunked one, on batch ids in no order, with one cloud that has
    # no points: minima and maxima equal numpy's, padded by 1e-6 in fp32 (BoundingBox.py:17-18)
    rng = np.random.default_rng(num_pts + batch)
    pts = rng.normal(size=(num_pts, 3)).astype(np.float32)
    ids = rng.integers(0, batch - 1, num_pts).astype(np.int32)          # cloud batch - 1 stays empty
    mn, mx = ops.bounding_box(t(pts), t(ids), batch)
    mn, mx = mn.cpu().numpy(), mx.cpu().numpy()
    for b in range(batch - 1):
        sel = pts[ids == b]
        if sel.shape[0] == 0:
            continue
        assert np.array_equal(mn[b], sel.min(axis=0) - np.float32(1e-6))
        assert np.array_equal(mx[b], sel.max(axis=0) + np.float32(1e-6))
    assert np.all(np.isposinf(mn[batch - 1])) and np.all(np.isneginf(mx[batch - 1]))


@pytest.mark.parametrize("use_table", [True, False])
def test_poisson_disk_from_the_grid_on_a_large_cloud_equals_the_list_version(ops, use_table):
    # The list-free selection at the size of a hierarchy's first level: a room plus two tight clusters, so that most
    # cells hold a few points and some hold hundreds (several rounds of 64 per cell, index ranges longer than the 64
    # flags a wavefront requests at once).  The neighbor-list version (itself checked against the oracle at small
    # sizes) must pick the same points.
    rng = np.random.default_rng(8)
    room = (synthetic.room(21, 230000) / 10.0).astype(np.float32)
    blobs = np.concatenate([rng.normal((0.3, 0.4, 0.1), 0.004, (9000, 3)),
                            rng.normal((0.71, 0.22, 0.05), 0.002, (6000, 3))]).astype(np.float32)
    pts = np.concatenate([room, blobs])[rng.permutation(room.shape[0] + blobs.shape[0])]
    ids = np.zeros(pts.shape[0], np.int32)
    ids[pts.shape[0] // 2:] = 1
    radius = 0.012
    g = gpu_neighborhood(ops, pts, ids, pts, ids, radius, 2)["dev"]
    table = ops.build_cell_table(g["skeys"], 2 * int(np.prod(g["nc"].tolist()))) if use_table else None
    sel = ops.poisson_disk_sampling_grid(g["spts"], g["skeys"], g["ds"], g["nc"], g["radii"], cell_table=table)
    neigh, ends = ops.find_neighbors_ex(g["spts"], g["skeys"], g["spts"], g["skeys"], g["ds"], g["nc"], g["radii"], 0)
    counts = torch.diff(ends, prepend=ends.new_zeros(1))
    assert int(counts.max()) > 200                       # the clusters are there
    want = ops.poisson_disk_sampling(g["skeys"], neigh, ends, g["nc"])
    assert sel.shape[0] > 1000 and torch.equal(sel, want)
    # the selection is a maximal independent set: no two selected points are neighbors, every other point has one
    chosen = torch.zeros(pts.shape[0], dtype=torch.bool, device=DEV)
    chosen[sel.reshape(-1)] = True
    pair_pt, pair_sample = neigh[:, 0].to(torch.int64), neigh[:, 1].to(torch.int64)
    both = chosen[pair_pt] & chosen[pair_sample] & (pair_pt != pair_sample)
    assert not bool(both.any())
    covered = torch.zeros(pts.shape[0], dtype=torch.bool, device=DEV)
    covered[pair_sample[chosen[pair_pt]]] = True
    assert bool(covered.all())


@pytest.mark.parametrize("pts_per_cloud,staged", [(2, False), (60, True)])
def test_one_call_pooling_with_more_clouds_than_the_kernels_write_to_the_host_themselves(ops, monkeypatch, pts_per_cloud,
                                                                                        staged):
    # 90 clouds are 270 box values, more than the one workgroup that may write them into the pinned block itself: the
    # one-call pooling then brings box and count over in copies (one staged copy of the boxes when the workspace has
    # room for them - not with two points per cloud -, else two) and the host waits for the event instead of polling.
    # Same tensors as the step-by-step route.
    import pccnn_lib_amd as lib
    from pccnn_lib_amd.pc import neighborhood, point_cloud, point_pooling
    batch = 90
    rng = np.random.default_rng(batch + pts_per_cloud)
    pts = rng.random((batch * pts_per_cloud, 3), dtype=np.float32)
    ids = np.repeat(np.arange(batch, dtype=np.int32), pts_per_cloud)
    n = pts.shape[0]
    assert (2 * batch * 12 + 4 <= 8 * n) == staged          # the library's own rule for the staged copy

    def run(one_call):
        for mod in (point_pooling, neighborhood, point_cloud):
            monkeypatch.setattr(mod, "ONE_CALL", one_call)
        pc = lib.pc.Pointcloud(pts, ids, device=DEV)
        pool = lib.pc.PointPooling(pc, 0.3)
        if one_call:
            assert pool.pending_ is not None and pool.pending_.polled is False
        out_pc = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
        box = lib.pc.BoundingBox(out_pc)
        fresh_min, fresh_max = ops.bounding_box(out_pc.pts_, out_pc.batch_ids_, batch)
        assert torch.equal(box.min_, fresh_min) and torch.equal(box.max_, fresh_max)
        assert np.array_equal(box.host()[0], fresh_min.cpu().numpy())
        assert np.array_equal(box.host()[1], fresh_max.cpu().numpy())
        return [pool.pooling_ids_, out_pc.pts_, out_pc.batch_ids_, box.min_, box.max_]

    a, b = run(False), run(True)
    assert a[0].shape[0] >= batch
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and torch.equal(x, y)


def test_box_of_many_clouds_in_six_dimensions_travels_in_copies(ops):
    # 50 clouds x 6 dimensions = 300 box values: the queued box does not write the pinned block from its kernels
    # (polled_out = 0); the copies and the event bring the same numbers as a read-back of the device tensors
    import pccnn_lib_amd as lib
    batch, per = 50, 40
    rng = np.random.default_rng(6)
    pts = rng.normal(size=(batch * per, 6)).astype(np.float32)
    ids = np.repeat(np.arange(batch, dtype=np.int32), per)
    mn, mx, fetch = ops.bounding_box_host_later(t(pts), t(ids), batch)
    assert fetch.polled is False
    host_min, host_max = fetch()
    assert np.array_equal(host_min, mn.cpu().numpy()) and np.array_equal(host_max, mx.cpu().numpy())
    exp_min = np.stack([pts[ids == b].min(axis=0) for b in range(batch)]) - np.float32(1e-6)
    assert np.array_equal(host_min, exp_min.astype(np.float32))
    box = lib.pc.BoundingBox(lib.pc.Pointcloud(pts, ids, device=DEV), p_with_host=True)
    assert np.array_equal(box.host()[0], box.min_.cpu().numpy()) and np.array_equal(box.host()[1], box.max_.cpu().numpy())
    # the small case for contrast: written by the kernels, polled
    small = ops.bounding_box_host_later(t(pts[:, :3].copy()), t(ids), batch)
    assert small[2].polled is True
    assert np.array_equal(small[2]()[0], small[0].cpu().numpy())


def test_polled_read_backs_fall_back_to_the_event_when_the_spin_limit_is_reached(ops, monkeypatch):
    # with a spin limit of zero the host gives up polling at once and waits for the event recorded behind the
    # kernels: same results
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(77, 3, 4000)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    want = lib.pc.PointPooling(pc, 0.07).pooling_ids_
    monkeypatch.setattr(ops, "SPIN_LIMIT", 0)
    pool = lib.pc.PointPooling(lib.pc.Pointcloud(pts, ids, device=DEV), 0.07)
    assert pool.pending_ is not None and pool.pending_.polled is True
    assert torch.equal(pool.pooling_ids_, want)
    mn, mx, fetch = ops.bounding_box_host_later(t(pts), t(ids), 3)
    assert np.array_equal(fetch()[0], mn.cpu().numpy()) and np.array_equal(fetch()[1], mx.cpu().numpy())
