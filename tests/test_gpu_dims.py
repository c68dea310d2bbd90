"""The path in 2, 4, 5 and 6 dimensions (the reference's own tests run in 2, 3, 4 and 6: unit_test/utest_*.ini).
Index results bit-exact against the oracle, which follows the reference's D-dimensional walk (offsets over all
dimensions but the last, key interval [k - 1, k + 1] inside the pillar of the first two); densities 1e-5, their
gradients 1e-4."""
import numpy as np
import pytest
import torch

from tests.gpu_helpers import DEV, gpu_neighborhood, relerr, t

pytestmark = pytest.mark.gpu

# (dimensions, clouds, points per cloud, radius): sparse in high dimensions, so the radius grows with D
CASES = [(2, 4, 1500, 0.05), (2, 2, 300, 0.3), (4, 3, 1200, 0.25), (5, 2, 1000, 0.4), (6, 2, 900, 0.5),
         (6, 1, 200, 1.0)]


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _cloud(dims, batch, num_pts, seed):
    rng = np.random.default_rng(seed)
    pts = rng.uniform(0.0, 1.0, (batch * num_pts, dims)).astype(np.float32)
    # squeeze every second cloud along the last axis so that boxes and grids differ between clouds
    ids = np.repeat(np.arange(batch, dtype=np.int32), num_pts)
    pts[ids % 2 == 1, -1] *= np.float32(0.5)
    return pts, ids


def _check_index(oracle, got, exp):
    for name in ("aabb_min", "aabb_max", "num_cells", "keys", "perm", "sorted_keys", "sorted_pts", "grid_ds",
                 "sample_keys", "ends"):
        assert np.array_equal(np.asarray(got[name]), np.asarray(exp[name])), name
    assert np.array_equal(oracle.canonical_pairs(got["neighbors"]), oracle.canonical_pairs(exp["neighbors"]))
    assert np.array_equal(oracle.canonical_pairs(got["neigh_sorted"]), oracle.canonical_pairs(exp["neigh_sorted"]))


@pytest.mark.parametrize("dims,batch,num_pts,radius", CASES)
def test_neighborhood_bit_exact(ops, oracle, dims, batch, num_pts, radius):
    pts, ids = _cloud(dims, batch, num_pts, 100 + dims)
    exp = oracle.neighborhood(pts, ids, pts, ids, radius)
    for use_order in (True, False):
        got = gpu_neighborhood(ops, pts, ids, pts, ids, radius, batch, use_order=use_order)
        _check_index(oracle, got, exp)
    # Brute force: the walk loses no pair.  Beyond three dimensions the reference takes the last dimension as the key
    # interval [k - 1, k + 1] inside a pillar that also spans dimensions 2 .. D-2, so at the first / last cell of the
    # last dimension the interval reaches into the neighbouring row of the pillar (find_ranges_grid_ds.cu:100-105).
    # With three or more cells along the last dimension that row is too far away to hold a neighbor; with two it is a
    # true neighbor cell that another offset visits as well, and the reference lists such pairs twice.  Oracle and
    # HIP path reproduce that; the set of distinct pairs is the brute-force set in every case.
    bf, bf_ends = oracle.brute_force_neighbors(pts, ids, pts, ids, np.full(dims, radius, np.float32))
    canon = oracle.canonical_pairs(exp["neighbors"])
    keep = np.ones(canon.shape[0], bool)
    keep[1:] = np.any(canon[1:] != canon[:-1], axis=1)
    assert np.array_equal(canon[keep], oracle.canonical_pairs(bf))
    if dims <= 3 or int(exp["num_cells"][-1]) >= 3:
        assert np.array_equal(exp["ends"], bf_ends)


@pytest.mark.parametrize("dims,batch,num_pts,radius", [(2, 3, 2000, 0.04), (4, 2, 2500, 0.22)])
def test_drop_in_find_neighbors_above_the_sorting_threshold(ops, oracle, dims, batch, num_pts, radius):
    # more than 4096 samples: the reference-signature op sorts the samples by itself; the per-cell start table is a
    # 3-dimensional structure and must stay out of it
    pts, ids = _cloud(dims, batch, num_pts, 500 + dims)
    assert pts.shape[0] > 4096
    exp = oracle.neighborhood(pts, ids, pts, ids, radius)
    g = gpu_neighborhood(ops, pts, ids, pts, ids, radius, batch)
    d = g["dev"]
    neigh, ends = ops.find_neighbors(d["spts"], d["skeys"], d["samples"], t(g["sample_keys"]), d["ds"], d["nc"],
                                     d["radii"], 0)
    assert np.array_equal(ends.cpu().numpy(), exp["ends"])
    assert np.array_equal(oracle.canonical_pairs(neigh.cpu().numpy()), oracle.canonical_pairs(exp["neigh_sorted"]))


@pytest.mark.parametrize("dims,batch,num_pts,radius", [(2, 3, 800, 0.1), (4, 2, 900, 0.3), (6, 2, 700, 0.6)])
def test_distinct_samples_and_cap(ops, oracle, dims, batch, num_pts, radius):
    pts, ids = _cloud(dims, batch, num_pts, 200 + dims)
    rng = np.random.default_rng(dims)
    pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
    smp, sids = (pts[pick] + np.float32(0.004)).astype(np.float32), ids[pick]
    for cap in (0, 5):
        exp = oracle.neighborhood(pts, ids, smp, sids, radius, max_neighbors=cap)
        got = gpu_neighborhood(ops, pts, ids, smp, sids, radius, batch, max_neighbors=cap)
        assert np.array_equal(got["ends"], exp["ends"])
        # the capped subset depends on the walk order, so the lists must agree pair for pair
        assert np.array_equal(got["neigh_sorted"], exp["neigh_sorted"])
        assert np.array_equal(got["neighbors"], exp["neighbors"])


@pytest.mark.parametrize("dims,batch,num_pts,radius", [(2, 2, 1000, 0.08), (4, 2, 800, 0.3), (6, 2, 600, 0.6)])
def test_pdf_and_gradients(ops, oracle, dims, batch, num_pts, radius):
    pts, ids = _cloud(dims, batch, num_pts, 300 + dims)
    got = gpu_neighborhood(ops, pts, ids, pts, ids, radius, batch)
    d = got["dev"]
    bw = np.full(dims, 0.25 * radius, np.float32)
    for manifold in (dims, 2):
        pdf = ops.compute_pdf(manifold, t(bw), d["pts"], d["neigh"], d["ends"])
        exp = oracle.compute_pdf(manifold, bw, pts, got["neighbors"], got["ends"])
        assert relerr(pdf.cpu().numpy(), exp) < 1e-5
        spdf = ops.compute_pdf_sorted(manifold, t(bw), d["spts"], d["pts"], t(got["neigh_sorted"]), d["ends"])
        assert relerr(spdf.cpu().numpy(), exp) < 1e-5
    g = np.random.default_rng(dims).normal(size=pts.shape[0]).astype(np.float32)
    grads = ops.compute_pdf_grads(dims, t(bw), d["pts"], d["neigh"], d["ends"], t(g))
    exp_g = oracle.compute_pdf_grads(dims, bw, pts, got["neighbors"], got["ends"], g)
    assert tuple(grads.shape) == pts.shape and relerr(grads.cpu().numpy(), exp_g) < 1e-4


@pytest.mark.parametrize("dims,batch,num_pts,radius", [(2, 3, 1500, 0.05), (4, 2, 1000, 0.3), (6, 2, 800, 0.6)])
def test_poisson_disk(ops, oracle, dims, batch, num_pts, radius):
    pts, ids = _cloud(dims, batch, num_pts, 400 + dims)
    exp = oracle.neighborhood(pts, ids, pts, ids, radius)
    e_neigh, e_ends = oracle.find_neighbors(exp["sorted_pts"], exp["sorted_keys"], exp["sorted_pts"],
                                            exp["sorted_keys"], exp["grid_ds"], exp["num_cells"], exp["radii"])
    e_sel = oracle.poisson_disk_sampling(exp["sorted_keys"], e_neigh, e_ends, exp["num_cells"])
    g = gpu_neighborhood(ops, pts, ids, pts, ids, radius, batch)["dev"]
    neigh, ends = ops.find_neighbors_ex(g["spts"], g["skeys"], g["spts"], g["skeys"], g["ds"], g["nc"], g["radii"], 0)
    sel = ops.poisson_disk_sampling(g["skeys"], neigh, ends, g["nc"])
    assert np.array_equal(sel.cpu().numpy(), e_sel)
    # the defining property, per cloud: selected points are at least one radius apart
    chosen = exp["sorted_pts"][e_sel[:, 0]].astype(np.float64)
    cid = ids[exp["perm"]][e_sel[:, 0]]
    for b in range(batch):
        q = chosen[cid == b]
        dist = np.linalg.norm(q[:, None] - q[None], axis=-1) + np.eye(q.shape[0]) * 1e9
        assert dist.min() >= radius * (1 - 1e-6)


def test_object_api_in_two_dimensions(oracle):
    # Pointcloud / Grid / Neighborhood / PointPooling / compute_pdf on planar clouds
    import pccnn_lib_amd as lib
    pts, ids = _cloud(2, 3, 2000, 7)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    radii = torch.full((2,), 0.05, device=DEV)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    exp = oracle.neighborhood(pts, ids, pts, ids, 0.05)
    assert np.array_equal(oracle.canonical_pairs(nbh.neighbors_.cpu().numpy()), oracle.canonical_pairs(exp["neighbors"]))
    assert np.array_equal(nbh.start_ids_.cpu().numpy(), exp["ends"])
    pc.compute_pdf(np.full(2, 0.02, np.float32))
    unnorm, norm, _ = oracle.pointcloud_pdf(pts, ids, 0.02)
    assert relerr(pc.pts_unnorm_pdf_.cpu().numpy(), unnorm) < 1e-5
    assert relerr(pc.pts_pdf_.cpu().numpy(), norm) < 1e-5
    pool = lib.pc.PointPooling(pc, radii)
    sel = pool.pooling_ids_.cpu().numpy().reshape(-1)
    q = pts[sel][ids[sel] == 1].astype(np.float64)
    dist = np.linalg.norm(q[:, None] - q[None], axis=-1) + np.eye(q.shape[0]) * 1e9
    assert dist.min() >= 0.05 * (1 - 1e-6)


@pytest.mark.parametrize("distinct", [False, True])
def test_planar_kpconv_and_mcconv(ops, oracle, distinct):
    # The reference's convolution tests also run in 2 dimensions (unit_test/utest_kpconv.ini, utest_mcconv.ini).
    # Planar clouds go through the 3-D kernels with a zero third coordinate; results against the oracle's 2-D formulas.
    pts, ids = _cloud(2, 2, 1200, 9)
    rng = np.random.default_rng(9)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    nb = gpu_neighborhood(ops, pts, ids, smp, sids, 0.08, 2)
    neigh, ends, radii, d = nb["neighbors"], nb["ends"], nb["radii"], nb["dev"]
    c_in, c_out, k = 16, 24, 16
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    # KPConv: centre + 15 directions on the circle, normalised like the layer does
    ang = 2 * np.pi * np.arange(k - 1) / (k - 1)
    kp = np.concatenate([np.zeros((1, 2)), np.stack([np.cos(ang), np.sin(ang)], 1)]).astype(np.float32) / np.float32(2.0)
    sigma = 0.5
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    args = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    host = (pts, feats, smp, neigh, ends, radii, kp, sigma, w)
    assert relerr(ops.kp_conv(*args).cpu().numpy(), oracle.kpconv(*host)) < 1e-5
    grads = ops.kp_conv_grads(*args, t(g))
    for got, e, name in zip(grads, oracle.kpconv_grads(*host, g), ("dW", "dFeat", "dKernelPts", "dPts", "dSamples")):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < 1e-4, name
    assert relerr(ops.kp_conv_weight_var(*args[:-1]).cpu().numpy(), oracle.kpconv_weight_var(*host[:-1])) < 1e-4
    # MCConv
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    axis = rng.normal(0, np.sqrt(0.5), (2, k)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, k)).astype(np.float32)
    wm = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (1, k * c_in, c_out)).astype(np.float32)
    margs = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(wm))
    mhost = (pts, pdf, feats, smp, neigh, ends, radii, axis, bias, wm)
    assert relerr(ops.mc_conv(*margs).cpu().numpy(), oracle.mcconv(*mhost)) < 1e-5
    names = ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")
    for got, e, name in zip(ops.mc_conv_grads(*margs, t(g)), oracle.mcconv_grads(*mhost, g), names):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < 1e-4, name


def test_planar_layers(oracle):
    import pccnn_lib_amd as lib
    pts, ids = _cloud(2, 2, 1500, 21)
    rng = np.random.default_rng(21)
    feats = rng.normal(size=(pts.shape[0], 8)).astype(np.float32)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV, requires_grad=True)
    pc.compute_pdf(np.full(2, 0.02, np.float32))
    torch.manual_seed(3)
    kp_layer = lib.pc.layers.KPConv(2, 8, 12, 16).to(DEV)
    mc_layer = lib.pc.layers.MCConv(2, 8, 12, 8).to(DEV)
    tf = t(feats).requires_grad_(True)
    out_kp, nbh = kp_layer(pc, pc, tf, 0.06)
    out_mc = mc_layer(pc, pc, tf, 0.06, nbh)
    (out_kp.sum() + out_mc.sum()).backward()
    p = lambda x: x.detach().cpu().numpy()
    radii = np.full(2, 0.06, np.float32)
    nb = (p(nbh.neighbors_), p(nbh.start_ids_))
    exp = oracle.kpconv(pts, feats, pts, nb[0], nb[1], radii, p(kp_layer.kernel_pts_), float(kp_layer.sigma_.item()),
                        p(kp_layer.conv_weights_))
    assert relerr(p(out_kp), exp) < 1e-5
    pdf = p(pc.pts_unnorm_pdf_ * torch.prod(t(radii)))
    exp = oracle.mcconv(pts, pdf, feats, pts, nb[0], nb[1], radii, p(mc_layer.proj_axis_), p(mc_layer.proj_bias_),
                        p(mc_layer.conv_weights_))
    assert relerr(p(out_mc), exp) < 1e-5
    assert tuple(pc.pts_.grad.shape) == pts.shape and bool(torch.isfinite(pc.pts_.grad).all())
    assert tuple(tf.grad.shape) == feats.shape


def _kernel_points(dims, k):
    from pccnn_lib_amd.pc.layers.kernel_points import kernel_points
    kp = kernel_points(dims, k)
    return (kp / (2.0 * np.linalg.norm(kp, axis=1).max())).astype(np.float32)


@pytest.mark.parametrize("dims,radius,distinct", [(4, 0.3, False), (4, 0.3, True), (5, 0.45, True), (6, 0.6, False)])
def test_convolutions_beyond_three_dimensions(ops, oracle, dims, radius, distinct):
    # The reference's convolution tests run in 4 dimensions too (unit_test/utest_kpconv.ini Test_4, utest_mcconv.ini
    # Test_4).  There the basis is evaluated per pair and the convolution runs on it as a caller-given basis.
    pts, ids = _cloud(dims, 2, 700, 500 + dims)
    rng = np.random.default_rng(dims)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    nb = gpu_neighborhood(ops, pts, ids, smp, sids, radius, 2)
    neigh, ends, radii, d = nb["neighbors"], nb["ends"], nb["radii"], nb["dev"]
    assert neigh.shape[0] > 4 * smp.shape[0]
    c_in, c_out, k = 12, 10, 16
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    kp, sigma = _kernel_points(dims, k), 0.5
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)

    def check(grads, expect, names):
        for got, e, name in zip(grads, expect, names):
            assert tuple(got.shape) == e.shape, name
            assert relerr(got.cpu().numpy(), e) < 1e-4, name

    # KPConv, against the oracle and against the closed form the reference's own test uses (unit_test/test_kpconv.py:63-80)
    args = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    host = (pts, feats, smp, neigh, ends, radii, kp, sigma, w)
    out = ops.kp_conv(*args).cpu().numpy()
    assert relerr(out, oracle.kpconv(*host)) < 1e-5
    diff = (pts[neigh[:, 0]].astype(np.float64) - smp[neigh[:, 1]]) / radii
    corr = np.clip(1.0 - np.linalg.norm(diff[:, None, :] - kp[None], axis=-1) / sigma, 0.0, 1.0)
    proj = np.zeros((smp.shape[0], c_in, k))
    np.add.at(proj, neigh[:, 1], feats[neigh[:, 0]][:, :, None] * corr[:, None, :])
    closed = proj.reshape(smp.shape[0], -1) @ w.astype(np.float64)
    assert relerr(out, closed) < 1e-5
    check(ops.kp_conv_grads(*args, t(g)), oracle.kpconv_grads(*host, g), ("dW", "dFeat", "dKernelPts", "dPts", "dSamples"))
    assert relerr(ops.kp_conv_weight_var(*args[:-1]).cpu().numpy(), oracle.kpconv_weight_var(*host[:-1])) < 1e-4
    part = ops.kp_conv_grads(*args, t(g), grad_mask=ops.GRAD_WEIGHTS | ops.GRAD_PTS)
    assert part[1] is None and part[2] is None
    full = oracle.kpconv_grads(*host, g)
    assert relerr(part[0].cpu().numpy(), full[0]) < 1e-4 and relerr(part[3].cpu().numpy(), full[3]) < 1e-4

    # MCConv with two MLPs
    axis = rng.normal(0, np.sqrt(1.0 / dims), (dims, k)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, k)).astype(np.float32)
    wm = rng.normal(0, np.sqrt(2.0 / (k * c_in)), (2, k * c_in // 2, c_out // 2)).astype(np.float32)
    margs = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(wm))
    mhost = (pts, pdf, feats, smp, neigh, ends, radii, axis, bias, wm)
    assert relerr(ops.mc_conv(*margs).cpu().numpy(), oracle.mcconv(*mhost)) < 1e-5
    check(ops.mc_conv_grads(*margs, t(g)), oracle.mcconv_grads(*mhost, g),
          ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples"))
    assert relerr(ops.mc_conv_weight_var(*margs[:-1]).cpu().numpy(), oracle.mcconv_weight_var(*mhost[:-1])) < 1e-4
    out16 = ops.mc_conv(*margs, contraction="bf16").cpu().numpy()
    assert relerr(out16, oracle.mcconv(*mhost, contraction="bf16")) < 3e-3

    # KPConvN and PCCNN through the generic entry points
    nargs = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    assert relerr(ops.kp_conv_n(*nargs).cpu().numpy(),
                  oracle.kpconvn(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma, w)) < 1e-5
    check(ops.kp_conv_n_grads(*nargs, t(g)), oracle.kpconvn_grads(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma, w, g),
          ("dW", "dFeat", "dKernelPts", "dPts", "dSamples"))
    var = ops.kp_conv_n_weight_var(*nargs[:-1])
    exp = oracle.kpconvn_weight_var(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma)
    assert abs(float(var) - float(exp)) < 1e-4 * abs(float(exp))
    gargs = (d["pts"], t(feats), t(pdf), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), 0.35, t(w))
    assert relerr(ops.pccnn(*gargs).cpu().numpy(),
                  oracle.pccnn(pts, feats, pdf, smp, neigh, ends, radii, kp, 0.35, w)) < 1e-5
    check(ops.pccnn_grads(*gargs, t(g)), oracle.pccnn_grads(pts, feats, pdf, smp, neigh, ends, radii, kp, 0.35, w, g),
          ("dW", "dFeat", "dKernelPts", "dPdf", "dPts", "dSamples"))

    # PointConv's basis op
    bargs = (d["pts"], d["radii"], d["samples"], d["neigh"], t(axis), t(bias))
    exp_basis, _ = oracle.pointconv_basis(pts, radii, smp, neigh, axis, bias)
    assert relerr(ops.point_conv_basis(*bargs).cpu().numpy(), exp_basis) < 1e-5
    gb = rng.normal(size=exp_basis.shape).astype(np.float32)
    check(ops.point_conv_basis_grads(*bargs, t(gb)), oracle.pointconv_basis_grads(pts, radii, smp, neigh, axis, bias, gb),
          ("dPts", "dSamples", "dAxis", "dBias"))

    # spherical bins need three coordinates
    edges = t(np.array([0.5, 1.0], np.float32))
    with pytest.raises(RuntimeError):
        ops.sph_conv(d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], edges, edges, edges,
                     t(rng.normal(size=(9 * c_in, c_out)).astype(np.float32)))


def test_empty_neighborhood_in_four_dimensions(ops):
    pts = t(np.random.default_rng(0).uniform(size=(50, 4)).astype(np.float32))
    feats = torch.ones((50, 4), device=DEV)
    none = torch.zeros((0, 2), dtype=torch.int32, device=DEV)
    ends = torch.zeros((50,), dtype=torch.int32, device=DEV)
    radii = torch.full((4,), 0.1, device=DEV)
    kp = t(_kernel_points(4, 8))
    w = torch.ones((8 * 4, 3), device=DEV)
    assert float(ops.kp_conv(pts, feats, pts, none, ends, radii, kp, 0.5, w).abs().max()) == 0.0
    grads = ops.kp_conv_grads(pts, feats, pts, none, ends, radii, kp, 0.5, w, torch.ones((50, 3), device=DEV))
    assert all(float(x.abs().max()) == 0.0 for x in grads)
    assert tuple(grads[3].shape) == (50, 4) and tuple(grads[2].shape) == (8, 4)


def test_layers_in_four_dimensions(oracle):
    # the shape of the reference's 4-D cases: unit_test/utest_kpconv.ini Test_4, utest_mcconv.ini Test_4
    import pccnn_lib_amd as lib
    pts, ids = _cloud(4, 4, 250, 33)
    rng = np.random.default_rng(33)
    feats = rng.normal(size=(pts.shape[0], 32)).astype(np.float32)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV, requires_grad=True)
    pc.compute_pdf(np.full(4, 0.1, np.float32))
    torch.manual_seed(5)
    kp_layer = lib.pc.layers.KPConv(4, 32, 4, 16).to(DEV)
    mc_layer = lib.pc.layers.MCConv(4, 32, 4, 8).to(DEV)
    tf = t(feats).requires_grad_(True)
    out_kp, nbh = kp_layer(pc, pc, tf, 0.25)
    out_mc = mc_layer(pc, pc, tf, 0.25, nbh)
    (out_kp.sum() + out_mc.sum()).backward()
    p = lambda x: x.detach().cpu().numpy()
    radii = np.full(4, 0.25, np.float32)
    neigh, ends = p(nbh.neighbors_), p(nbh.start_ids_)
    kp, sigma, w = p(kp_layer.kernel_pts_), float(kp_layer.sigma_.item()), p(kp_layer.conv_weights_)
    assert relerr(p(out_kp), oracle.kpconv(pts, feats, pts, neigh, ends, radii, kp, sigma, w)) < 1e-5
    pdf = p(pc.pts_unnorm_pdf_ * torch.prod(t(radii)))
    exp = oracle.mcconv(pts, pdf, feats, pts, neigh, ends, radii, p(mc_layer.proj_axis_), p(mc_layer.proj_bias_),
                        p(mc_layer.conv_weights_))
    assert relerr(p(out_mc), exp) < 1e-5
    ones = np.ones((pts.shape[0], 4), np.float32)
    e_kp = oracle.kpconv_grads(pts, feats, pts, neigh, ends, radii, kp, sigma, w, ones)
    assert relerr(p(kp_layer.conv_weights_.grad), e_kp[0]) < 1e-4
    assert tuple(pc.pts_.grad.shape) == pts.shape and bool(torch.isfinite(pc.pts_.grad).all())
    assert tuple(tf.grad.shape) == feats.shape
