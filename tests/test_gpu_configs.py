"""The baseline configurations at their full sizes.

The oracle needs minutes for a whole batch, but clouds of a batch never interact (the batch id is the top digit of
the cell key), so everything that is per point or per sample -- neighbor lists, densities, outputs, feature and point
gradients -- is checked for single clouds of the full-size run against the oracle run on those clouds alone.
Quantities summed over the whole batch (weight and basis-parameter gradients) are checked through linearity: the
full-batch result must equal the sum of the HIP results of the single clouds, and the single-cloud results are
checked against the oracle."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, relerr, t

pytestmark = pytest.mark.gpu

FWD_TOL = 1e-5
GRAD_TOL = 1e-4
# bf16 contraction against the oracle with the same operand rounding: an entry of the fp32 projection that sits on a
# bf16 rounding boundary may round the other way (one bf16 step of one term of a sum of K*Cin), which is what the
# output tolerance leaves room for; the gradients are sums over many samples and meet the fp32 bar.
BF16_OUT_TOL = 1e-3
BF16_GRAD_TOL = 1e-4


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _cloud_slices(ids, nbh_neigh, nbh_ends, cloud, num_pts):
    """Rows of one cloud in a batch of equally sized clouds, and its pair list re-based to local indices."""
    lo, hi = cloud * num_pts, (cloud + 1) * num_pts
    e = nbh_ends
    p_lo = int(e[lo - 1]) if lo > 0 else 0
    p_hi = int(e[hi - 1])
    neigh = nbh_neigh[p_lo:p_hi] - lo
    ends = e[lo:hi] - p_lo
    return slice(lo, hi), neigh.astype(np.int32), ends.astype(np.int32)


def test_config2_mcconv_16x4096(ops, oracle):
    # Batch 16 x 4096 primitives, radius 0.05, KDE bandwidth 0.01, MCConv hidden 16, 64 -> 128, fp32;
    # gradients w.r.t. features and weights (and, beyond the configuration, the basis parameters).
    import pccnn_lib_amd as lib
    batch, num_pts, c_in, c_out, hidden = 16, 4096, 64, 128, 16
    pts, ids = synthetic.primitives(2, batch, num_pts)
    rng = np.random.default_rng(2)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1.0 / 3.0), (3, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, hidden)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (hidden * c_in)), (1, hidden * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    radii = torch.full((3,), 0.05, device=DEV)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pc.compute_pdf(np.full(3, 0.01, np.float32))
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    pdf_t = (pc.pts_unnorm_pdf_ * torch.prod(radii)).contiguous()
    args = (pc.pts_, pdf_t, t(feats), pc.pts_, nbh.neighbors_, nbh.start_ids_, radii, t(axis), t(bias), t(w))
    out = ops.mc_conv(*args).cpu().numpy()
    grads = [x.cpu().numpy() for x in ops.mc_conv_grads(*args, t(g))]
    neigh, ends, pdf = nbh.neighbors_.cpu().numpy(), nbh.start_ids_.cpu().numpy(), pdf_t.cpu().numpy()
    unnorm = pc.pts_unnorm_pdf_.cpu().numpy()
    r = np.full(3, 0.05, np.float32)
    dw_sum, daxis_sum, dbias_sum = 0.0, 0.0, 0.0
    for cloud in range(batch):
        rows, ln, le = _cloud_slices(ids, neigh, ends, cloud, num_pts)
        sub = (pc.pts_[rows].contiguous(), pdf_t[rows].contiguous(), t(feats[rows]), pc.pts_[rows].contiguous(),
               t(ln), t(le), radii, t(axis), t(bias), t(w))
        part = [x.cpu().numpy() for x in ops.mc_conv_grads(*sub, t(g[rows]))]
        dw_sum, daxis_sum, dbias_sum = dw_sum + part[0].astype(np.float64), daxis_sum + part[2], dbias_sum + part[3]
        if cloud in (0, batch - 1):
            zeros = np.zeros(num_pts, np.int32)
            nb = oracle.neighborhood(pts[rows], zeros, pts[rows], zeros, 0.05)
            assert np.array_equal(oracle.canonical_pairs(ln), oracle.canonical_pairs(nb["neighbors"]))
            assert np.array_equal(le, nb["ends"])
            o_unnorm, _, _ = oracle.pointcloud_pdf(pts[rows], zeros, 0.01)
            assert relerr(unnorm[rows], o_unnorm) < FWD_TOL
            host = (pts[rows], pdf[rows], feats[rows], pts[rows], ln, le, r, axis, bias, w)
            assert relerr(out[rows], oracle.mcconv(*host)) < FWD_TOL
            exp = oracle.mcconv_grads(*host, g[rows])
            assert relerr(grads[1][rows], exp[1]) < GRAD_TOL                  # dFeat rows of this cloud
            assert relerr(grads[4][rows], exp[4]) < GRAD_TOL                  # dPdf
            assert relerr(grads[5][rows] + grads[6][rows], exp[5] + exp[6]) < GRAD_TOL      # dPts + dSamples
            for i in (0, 2, 3):
                assert relerr(part[i], exp[i]) < GRAD_TOL                     # single-cloud dW, dAxis, dBias
    assert relerr(grads[0], dw_sum) < GRAD_TOL
    assert relerr(grads[2], daxis_sum) < GRAD_TOL
    assert relerr(grads[3], dbias_sum) < GRAD_TOL


def test_config3_kpconv_full_gradients_8x8192(ops, oracle):
    # Batch 8 x 8192 primitives, radius 0.04, 15 kernel points, 128 -> 256, fp32: forward plus gradients w.r.t.
    # features, weights and point positions (points are also the samples: the two position gradients add up).
    import pccnn_lib_amd as lib
    batch, num_pts, c_in, c_out, k = 8, 8192, 128, 256, 15
    pts, ids = synthetic.primitives(3, batch, num_pts)
    rng = np.random.default_rng(3)
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(2.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    radii = torch.full((3,), 0.04, device=DEV)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    args = (pc.pts_, t(feats), pc.pts_, nbh.neighbors_, nbh.start_ids_, radii, t(kp), sigma, t(w))
    out = ops.kp_conv(*args).cpu().numpy()
    grads = [x.cpu().numpy() for x in ops.kp_conv_grads(*args, t(g), mirror=nbh.mirror())]
    plain = [x.cpu().numpy() for x in ops.kp_conv_grads(*args, t(g))]         # same without the mirror index
    for a, b in zip(grads, plain):
        assert relerr(a, b) < GRAD_TOL
    neigh, ends = nbh.neighbors_.cpu().numpy(), nbh.start_ids_.cpu().numpy()
    r = np.full(3, 0.04, np.float32)
    dw_sum, dkp_sum = 0.0, 0.0
    for cloud in range(batch):
        rows, ln, le = _cloud_slices(ids, neigh, ends, cloud, num_pts)
        sub = (pc.pts_[rows].contiguous(), t(feats[rows]), pc.pts_[rows].contiguous(), t(ln), t(le), radii, t(kp),
               sigma, t(w))
        part = [x.cpu().numpy() for x in ops.kp_conv_grads(*sub, t(g[rows]))]
        dw_sum, dkp_sum = dw_sum + part[0].astype(np.float64), dkp_sum + part[2].astype(np.float64)
        if cloud == batch - 1:
            zeros = np.zeros(num_pts, np.int32)
            nb = oracle.neighborhood(pts[rows], zeros, pts[rows], zeros, 0.04)
            assert np.array_equal(oracle.canonical_pairs(ln), oracle.canonical_pairs(nb["neighbors"]))
            host = (pts[rows], feats[rows], pts[rows], ln, le, r, kp, sigma, w)
            assert relerr(out[rows], oracle.kpconv(*host)) < FWD_TOL
            exp = oracle.kpconv_grads(*host, g[rows])
            assert relerr(grads[1][rows], exp[1]) < GRAD_TOL
            assert relerr(grads[3][rows] + grads[4][rows], exp[3] + exp[4]) < GRAD_TOL
            assert relerr(part[0], exp[0]) < GRAD_TOL
            assert relerr(part[2], exp[2]) < GRAD_TOL
    assert relerr(grads[0], dw_sum) < GRAD_TOL
    assert relerr(grads[2], dkp_sum) < GRAD_TOL


def test_config4_million_point_scene(ops, oracle):
    # One room of 1 000 000 points, cell = radius = 0.05 m: keys, grid, neighbors, density.  Size-independent
    # properties on the whole result, and the oracle's own answer for the samples of a few thousand cells.
    import pccnn_lib_amd as lib
    n = 1000000
    pts = synthetic.room(4, n)
    ids = np.zeros(n, np.int32)
    radii = torch.full((3,), 0.05, device=DEV)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    grid = nbh.grid_
    keys, perm = grid.sorted_cell_ids_.cpu().numpy(), grid.sorted_ids_.cpu().numpy()
    assert np.array_equal(np.sort(perm), np.arange(n))
    assert np.all(np.diff(keys) >= 0) and np.array_equal(keys, grid.cell_ids_.cpu().numpy()[perm])
    neigh, ends = nbh.neighbors_.cpu().numpy(), nbh.start_ids_.cpu().numpy()
    counts = np.diff(ends, prepend=0)
    assert ends[-1] == neigh.shape[0] and counts.min() >= 1
    assert np.array_equal(neigh[:, 1], np.repeat(np.arange(n, dtype=np.int32), counts))
    d = np.linalg.norm(pts[neigh[:, 0]].astype(np.float64) - pts[neigh[:, 1]].astype(np.float64), axis=1)
    assert d.max() < 0.05 * (1 + 1e-5)
    fwd = neigh[:, 0].astype(np.int64) * n + neigh[:, 1]
    bwd = neigh[:, 1].astype(np.int64) * n + neigh[:, 0]
    assert np.array_equal(np.sort(fwd), np.sort(bwd))                             # symmetric
    assert np.count_nonzero(neigh[:, 0] == neigh[:, 1]) == n                        # every point finds itself
    # brute force (the oracle's O(N*M) search with the kernel's predicate) for 3000 samples spread over the scene,
    # against the points of a box that contains their whole neighborhoods
    pick = np.sort(np.random.default_rng(0).choice(n, 3000, replace=False))
    exp_counts = np.zeros(pick.shape[0], np.int64)
    tree_pts = pts.astype(np.float32)
    order = np.argsort(tree_pts[:, 0], kind="stable")
    xs = tree_pts[order, 0]
    for i, s in enumerate(pick):
        lo, hi = np.searchsorted(xs, [pts[s, 0] - 0.051, pts[s, 0] + 0.051])
        cand = order[lo:hi]
        bf, _ = oracle.brute_force_neighbors(pts[s:s + 1], ids[:1], pts[cand], ids[cand], np.full(3, 0.05, np.float32))
        got = np.sort(neigh[ends[s] - counts[s]:ends[s], 0])
        assert np.array_equal(got, np.sort(cand[bf[:, 0]])), "sample %d" % s
        exp_counts[i] = bf.shape[0]
    assert np.array_equal(counts[pick], exp_counts)
    # density over the search the reference prescribes (radius 4 x bandwidth, at most 300 neighbors): for the same
    # samples, the closed form in float64 over their brute-force neighbors within 4 bandwidths (no sample of this
    # scene reaches the cap)
    bw = 0.01
    pc.compute_pdf(np.full(3, bw, np.float32))
    pdf = pc.pts_unnorm_pdf_.cpu().numpy()
    assert np.all(np.isfinite(pdf)) and pdf.min() > 0.0
    const = (1.0 / bw) ** 3 / np.power(2.0 * 3.1415, 1.5)
    for s in pick[:500]:
        lo, hi = np.searchsorted(xs, [pts[s, 0] - 0.041, pts[s, 0] + 0.041])
        cand = order[lo:hi]
        bf, _ = oracle.brute_force_neighbors(pts[s:s + 1], ids[:1], pts[cand], ids[cand], np.full(3, 4 * bw, np.float32))
        assert bf.shape[0] <= 300
        diff = (pts[cand[bf[:, 0]]].astype(np.float32) - pts[s].astype(np.float32)) * np.float32(1.0 / bw)
        exp = const * np.exp(-0.5 * (diff.astype(np.float64) ** 2).sum(axis=1)).sum()
        assert abs(pdf[s] - exp) <= 2e-5 * exp, "sample %d" % s


def test_config5_hierarchy_8x100k_against_the_oracle(oracle):
    # Batch 8 x 100 000 room points (normalised by the longest side), four Poisson-disk levels with radii
    # 0.025 / 0.05 / 0.1 / 0.2, each followed by neighbor search, density and an MCConv 8 -> 32 -> 64 -> 128 -> 256
    # with bf16 contraction operands; forward and backward in one pass at the configuration's size.
    # Level 0 (800 000 points): Poisson-disk properties at full size, and its last cloud against the oracle
    # (selection, pair list, density, output, gradients).  Levels 1 - 3 (34 123 / 6 844 / 1 514 points): the whole
    # batch against the oracle - selected ids and pair lists bit-exact, density, outputs and every gradient.
    import pccnn_lib_amd as lib
    from pccnn_lib_amd import pccnn_lib_ops as ops
    batch, num_pts = 8, 100000
    pts = np.concatenate([synthetic.room(70 + b, num_pts) / 10.0 for b in range(batch)]).astype(np.float32)
    ids = np.repeat(np.arange(batch, dtype=np.int32), num_pts)
    rng = np.random.default_rng(5)
    torch.manual_seed(5)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    feats = t(rng.normal(size=(pts.shape[0], 8)).astype(np.float32)).requires_grad_(True)
    cur_pc, cur_feats, c_in = pc, feats, 8
    p = lambda x: x.detach().cpu().numpy()
    levels = []
    for level, (radius, c_out) in enumerate(zip((0.025, 0.05, 0.1, 0.2), (32, 64, 128, 256))):
        r3 = torch.full((3,), radius, device=DEV)
        pool = lib.pc.PointPooling(cur_pc, r3)
        sel = p(pool.pooling_ids_).reshape(-1)
        hp, hi = p(cur_pc.pts_), p(cur_pc.batch_ids_)
        assert np.unique(sel).shape[0] == sel.shape[0] and sel.min() >= 0 and sel.max() < hp.shape[0]
        # Poisson-disk property on one cloud: no two selected points closer than the radius, and every point of the
        # cloud has a selected point within the radius (checked on a sample of the cloud)
        b = batch - 1
        q = hp[sel][hi[sel] == b].astype(np.float64)
        chunk = q[:: max(1, q.shape[0] // 1500)]
        dist = np.linalg.norm(chunk[:, None] - q[None], axis=-1)
        dist[dist == 0.0] = np.inf
        assert dist.min() >= radius * (1 - 1e-6)
        probe = hp[hi == b][:: max(1, int((hi == b).sum()) // 1500)].astype(np.float64)
        assert np.linalg.norm(probe[:, None] - q[None], axis=-1).min(axis=1).max() < radius * (1 + 1e-6)
        out_pc = lib.pc.Pointcloud(pool.pool_tensor(cur_pc.pts_), pool.pool_tensor(cur_pc.batch_ids_))
        cur_pc.compute_pdf(np.full(3, 0.2 * radius, np.float32))
        layer = lib.pc.layers.MCConv(3, c_in, c_out, 8).to(DEV)
        layer.contraction_ = "bf16"
        if cur_feats is not feats:
            cur_feats.retain_grad()
        out, nbh = layer(cur_pc, out_pc, cur_feats, 2.0 * radius)
        assert bool(torch.isfinite(out).all()) and out.shape == (out_pc.pts_.shape[0], c_out)
        ends = p(nbh.start_ids_)
        assert ends[-1] == nbh.neighbors_.shape[0] and np.all(np.diff(ends, prepend=0) >= 1)
        out.retain_grad()
        levels.append(dict(pc_in=cur_pc, pc_out=out_pc, layer=layer, feats=cur_feats, out=out, nbh=nbh, sel=sel,
                           pool_radius=radius, radius=2 * radius))
        cur_pc, cur_feats, c_in = out_pc, torch.nn.functional.leaky_relu(out, 0.2), c_out
    out.sum().backward()
    assert feats.grad is not None and bool(torch.isfinite(feats.grad).all()) and float(feats.grad.abs().max()) > 0.0

    def expected_selection(hp, hi, radius):
        # pccnn_lib/pc/PointPooling.py:39-69 on the oracle: grid, self-neighborhood in sorted index space, selection,
        # original indices through the sort's permutation
        enb = oracle.neighborhood(hp, hi, hp, hi, radius)
        e_neigh, e_ends = oracle.find_neighbors(enb["sorted_pts"], enb["sorted_keys"], enb["sorted_pts"],
                                                enb["sorted_keys"], enb["grid_ds"], enb["num_cells"], enb["radii"])
        e_sel = oracle.poisson_disk_sampling(enb["sorted_keys"], e_neigh, e_ends, enb["num_cells"]).reshape(-1)
        return enb["perm"][e_sel].astype(np.int64)

    # Levels 1 - 3: the whole batch against the oracle.  The oracle takes the level's inputs (points, features, the
    # gradient that arrived at the level's output through the levels above it) from the pass itself.
    for level in (1, 2, 3):
        lv = levels[level]
        hp, hi = p(lv["pc_in"].pts_), p(lv["pc_in"].batch_ids_)
        hs, hsi = p(lv["pc_out"].pts_), p(lv["pc_out"].batch_ids_)
        assert np.array_equal(lv["sel"], expected_selection(hp, hi, lv["pool_radius"])), level
        assert np.array_equal(hs, hp[lv["sel"]]) and np.array_equal(hsi, hi[lv["sel"]])
        nb = oracle.neighborhood(hp, hi, hs, hsi, lv["radius"], batch_size=batch)
        neigh, ends = p(lv["nbh"].neighbors_), p(lv["nbh"].start_ids_)
        assert np.array_equal(ends, nb["ends"]), level
        assert np.array_equal(oracle.canonical_pairs(neigh), oracle.canonical_pairs(nb["neighbors"])), level
        unnorm, norm, _ = oracle.pointcloud_pdf(hp, hi, 0.2 * lv["pool_radius"])
        assert relerr(p(lv["pc_in"].pts_unnorm_pdf_), unnorm) < 1e-5, level
        assert relerr(p(lv["pc_in"].pts_pdf_), norm) < 1e-5, level
        radii = np.full(3, lv["radius"], np.float32)
        pdf = p(lv["pc_in"].pts_unnorm_pdf_ * torch.prod(t(radii)))
        layer = lv["layer"]
        host = (hp, pdf, p(lv["feats"]), hs, neigh, ends, radii, p(layer.proj_axis_), p(layer.proj_bias_),
                p(layer.conv_weights_))
        exp = oracle.mcconv(*host, contraction="bf16")
        assert relerr(p(lv["out"]), exp) < BF16_OUT_TOL, level
        exp_g = oracle.mcconv_grads(*host, p(lv["out"].grad), contraction="bf16")
        got_g = (layer.conv_weights_.grad, lv["feats"].grad, layer.proj_axis_.grad, layer.proj_bias_.grad)
        for got, e, name in zip(got_g, exp_g, ("dW", "dFeat", "dAxis", "dBias")):
            assert relerr(p(got), e) < BF16_GRAD_TOL, (level, name)

    # first level, last cloud, against the oracle (inputs of that cloud only)
    lv = levels[0]
    hp, hi = p(lv["pc_in"].pts_), p(lv["pc_in"].batch_ids_)
    hs, hsi = p(lv["pc_out"].pts_), p(lv["pc_out"].batch_ids_)
    b = batch - 1
    pin, sin = np.nonzero(hi == b)[0], np.nonzero(hsi == b)[0]
    z = lambda a: np.zeros(a.shape[0], np.int32)
    # the selection of a cloud depends on that cloud alone (cells are counted from the cloud's own box corner)
    own = lv["sel"][hi[lv["sel"]] == b] - pin[0]
    assert np.array_equal(own, expected_selection(hp[pin], z(pin), lv["pool_radius"]))
    nb = oracle.neighborhood(hp[pin], z(pin), hs[sin], z(sin), lv["radius"], batch_size=1)
    neigh, ends = p(lv["nbh"].neighbors_), p(lv["nbh"].start_ids_)
    p_lo = int(ends[sin[0] - 1]) if sin[0] > 0 else 0
    local = neigh[p_lo:int(ends[sin[-1]])] - np.array([pin[0], sin[0]], np.int32)
    assert np.array_equal(oracle.canonical_pairs(local), oracle.canonical_pairs(nb["neighbors"]))
    unnorm, _, _ = oracle.pointcloud_pdf(hp[pin], z(pin), 0.2 * lv["pool_radius"])
    assert relerr(p(lv["pc_in"].pts_unnorm_pdf_)[pin], unnorm) < 1e-5
    radii = np.full(3, lv["radius"], np.float32)
    pdf = p(lv["pc_in"].pts_unnorm_pdf_ * torch.prod(t(radii)))[pin]
    layer = lv["layer"]
    host = (hp[pin], pdf, p(lv["feats"])[pin], hs[sin], local.astype(np.int32), (ends[sin] - p_lo).astype(np.int32),
            radii, p(layer.proj_axis_), p(layer.proj_bias_), p(layer.conv_weights_))
    exp = oracle.mcconv(*host, contraction="bf16")
    assert relerr(p(lv["out"])[sin], exp) < BF16_OUT_TOL
    # Gradients of that cloud at the configuration's size.  The gradient that arrived at the first level's output
    # through the three levels above it is the oracle's input.  Clouds do not interact, so the feature-gradient
    # rows of the cloud in the end-to-end pass must be the oracle's; the weight gradient is summed over the batch,
    # so the cloud's own share comes from one more call of the op on the cloud's slice (same kernels, same sizes).
    g_out = p(lv["out"].grad)[sin]
    exp_g = oracle.mcconv_grads(*host, g_out, contraction="bf16")
    assert relerr(p(feats.grad)[pin], exp_g[1]) < BF16_GRAD_TOL
    got_g = ops.mc_conv_grads(*[t(a) for a in host], t(g_out), contraction="bf16")
    for i, name in ((0, "dW"), (1, "dFeat"), (2, "dAxis"), (3, "dBias"), (4, "dPdf")):
        assert relerr(p(got_g[i]), exp_g[i]) < BF16_GRAD_TOL, name


@pytest.mark.parametrize("kind", ["KPConv", "KPConvN"])
def test_kernel_point_layers_on_the_sorted_copy_equal_the_plain_run(monkeypatch, kind):
    # the same for the kernel-point layers (with and without the density)
    import pccnn_lib_amd as lib
    from pccnn_lib_amd.pc.layers import conv_base
    torch.manual_seed(4)
    pts = t(np.concatenate([synthetic.room(30 + b, 5000) / 10.0 for b in range(2)]).astype(np.float32))
    ids = t(np.repeat(np.arange(2, dtype=np.int32), 5000))
    layer = getattr(lib.pc.layers, kind)(3, 8, 16, 16).to(DEV)
    feats0 = torch.randn(pts.shape[0], 8, device=DEV)

    def run(min_points):
        monkeypatch.setattr(conv_base, "KEY_ORDER_MIN_POINTS", min_points)
        pc = lib.pc.Pointcloud(pts, ids)
        pc.compute_pdf(0.01)
        pool = lib.pc.PointPooling(pc, 0.05)
        pc_out = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
        feats = feats0.clone().requires_grad_(True)
        out, nbh = layer(pc, pc_out, feats, 0.1)
        grads = torch.autograd.grad(out.sum(), [feats, layer.conv_weights_])
        return out.detach(), grads, nbh

    out_a, grads_a, nbh_a = run(10 ** 9)
    out_b, grads_b, nbh_b = run(0)
    assert nbh_a.neighbors_key_order_ is None and nbh_b.neighbors_key_order_ is not None
    assert torch.equal(out_a, out_b)
    for ga, gb in zip(grads_a, grads_b):
        assert relerr(gb.cpu().numpy(), ga.cpu().numpy()) < 1e-5


@pytest.mark.parametrize("pooled", [True, False])
def test_mcconv_on_the_sorted_copy_of_a_large_cloud_equals_the_plain_run(monkeypatch, pooled):
    # From conv_base.KEY_ORDER_MIN_POINTS input points on, an MCConv layer that builds its own neighborhood keeps the
    # pair list in key order and runs on the grid's sorted copy of the cloud (features and densities permuted once).
    # With the threshold lowered: the same outputs (the sums run over the same pairs in the same order) and the same
    # gradients as the plain run, and `neighbors_` of the returned neighborhood is still the reference's list.
    import pccnn_lib_amd as lib
    from pccnn_lib_amd.pc.layers import conv_base
    torch.manual_seed(3)
    pts = t(np.concatenate([synthetic.room(20 + b, 6000) / 10.0 for b in range(3)]).astype(np.float32))
    ids = t(np.repeat(np.arange(3, dtype=np.int32), 6000))
    layer = lib.pc.layers.MCConv(3, 8, 32, 8).to(DEV)
    feats0 = torch.randn(pts.shape[0], 8, device=DEV)
    out_grads = torch.randn(1, 32, device=DEV)

    def run(min_points):
        monkeypatch.setattr(conv_base, "KEY_ORDER_MIN_POINTS", min_points)
        pc = lib.pc.Pointcloud(pts, ids)
        pc.compute_pdf(0.01)
        pc_out = pc
        if pooled:
            pool = lib.pc.PointPooling(pc, 0.05)
            pc_out = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
        feats = feats0.clone().requires_grad_(True)
        out, nbh = layer(pc, pc_out, feats, 0.1)
        grads = torch.autograd.grad((out * out_grads).sum(), [feats, layer.conv_weights_, layer.proj_axis_,
                                                               layer.proj_bias_])
        return out.detach(), grads, nbh

    out_a, grads_a, nbh_a = run(10 ** 9)
    out_b, grads_b, nbh_b = run(0)
    assert nbh_a.neighbors_key_order_ is None and nbh_b.neighbors_key_order_ is not None
    assert torch.equal(out_a, out_b)
    for ga, gb in zip(grads_a, grads_b):
        assert relerr(gb.cpu().numpy(), ga.cpu().numpy()) < 1e-5
    assert torch.equal(nbh_a.neighbors_, nbh_b.neighbors_) and torch.equal(nbh_a.start_ids_, nbh_b.start_ids_)


def test_projection_with_more_than_two_to_the_31_elements(ops):
    # Maximum sizes: 2.2 million samples x 64 features x 16 hidden units put 2.25e9 floats (9 GB) into the projection
    # and as many into its gradient, past what 32-bit element offsets reach.  No oracle runs at this size; the check
    # is that samples are independent: the convolution of the first and of the second part of the samples, run as two
    # smaller calls on re-based pair lists, must give the rows of the full call (forward) and gradients that add up
    # to the full call's (backward; summation order differs, hence the tolerance).
    import pccnn_lib_amd as lib
    n, c_in, hidden, c_out = 2_200_000, 64, 16, 32
    rng = np.random.default_rng(31)
    pts = t(rng.random((n, 3), dtype=np.float32))
    ids = torch.zeros(n, dtype=torch.int32, device=DEV)
    radii = torch.full((3,), 0.006, device=DEV)
    pc = lib.pc.Pointcloud(pts, ids)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    neigh, ends = nbh.neighbors_, nbh.start_ids_
    assert neigh.shape[0] > 2 * n                       # on average more than the point itself
    gen = torch.Generator(device=DEV).manual_seed(31)
    feats = torch.randn((n, c_in), device=DEV, generator=gen)
    pdf = torch.rand((n,), device=DEV, generator=gen) + 0.5
    axis = torch.randn((3, hidden), device=DEV, generator=gen) * 0.6
    bias = torch.randn((1, hidden), device=DEV, generator=gen) * 0.2
    w = torch.randn((1, hidden * c_in, c_out), device=DEV, generator=gen) * 0.03
    g = torch.randn((n, c_out), device=DEV, generator=gen)

    out, proj = ops.mc_conv(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, w, return_proj=True)
    assert proj.numel() > 2 ** 31
    full = ops.mc_conv_grads(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, w, g, proj=proj)
    del proj
    h = n // 2 + 12345
    cut = int(ends[h - 1])
    parts = []
    for lo, hi, p_lo, p_hi in ((0, h, 0, cut), (h, n, cut, neigh.shape[0])):
        nb = neigh[p_lo:p_hi].clone()
        nb[:, 1] -= lo
        en = (ends[lo:hi] - p_lo).contiguous()
        smp = pts[lo:hi].contiguous()
        o = ops.mc_conv(pts, pdf, feats, smp, nb, en, radii, axis, bias, w)
        assert torch.allclose(o, out[lo:hi], rtol=1e-6, atol=1e-6), (lo, hi)
        parts.append(ops.mc_conv_grads(pts, pdf, feats, smp, nb, en, radii, axis, bias, w, g[lo:hi].contiguous()))
        del o, nb, en, smp
    torch.cuda.synchronize()
    names = ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts")
    for i, name in enumerate(names):
        summed = parts[0][i] + parts[1][i]
        assert relerr(summed.cpu().numpy(), full[i].cpu().numpy()) < GRAD_TOL, name
    d_samples = torch.cat([parts[0][6], parts[1][6]])
    assert relerr(d_samples.cpu().numpy(), full[6].cpu().numpy()) < GRAD_TOL
