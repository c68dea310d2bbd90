"""HIP path vs the CPU oracle for the floating-point part of the path.  Tolerances: density and
convolution outputs 1e-5 relative (to the largest magnitude of the tensor), gradients 1e-4."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, mixed_close, relerr, t

pytestmark = pytest.mark.gpu

FWD_TOL = 1e-5
GRAD_TOL = 1e-4


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _cloud(models, batch, num_pts):
    pts = np.ascontiguousarray(models[:batch, :num_pts, :].reshape(-1, 3), np.float32)
    return pts, np.repeat(np.arange(batch, dtype=np.int32), num_pts)


# ------------------------------------------------------------------------------------ gemm

@pytest.mark.parametrize("rows,cols,inner,at,bt,split", [
    (256, 128, 64, 0, 0, 1), (300, 70, 45, 0, 0, 1), (128, 256, 32, 0, 1, 1), (77, 130, 19, 0, 1, 1),
    (128, 128, 4096, 1, 0, 8), (480, 40, 1000, 1, 0, 4), (129, 129, 17, 1, 1, 1), (1024, 128, 1024, 0, 0, 1),
    # full tiles in every layout (64-row and 128-row tiles of the kernel without bounds checks), with and without
    # a split of the reduction, and a reduction too short for that kernel
    (192, 384, 208, 0, 0, 1), (192, 384, 208, 1, 0, 1), (192, 384, 208, 0, 1, 1), (192, 384, 208, 1, 1, 1),
    (32768, 256, 192, 0, 0, 1), (32768, 128, 192, 1, 0, 1), (32768, 256, 192, 0, 1, 1), (32768, 128, 192, 1, 1, 1),
    (256, 256, 16384, 1, 0, 8), (1024, 128, 8192, 1, 0, 32), (32768, 256, 64, 0, 1, 1),
    # edge tiles read with whole 16-byte units (extents are multiples of the unit, not of the tile): the three
    # products of a small hierarchy level, forward, weight gradient (with a cut last split) and projection gradient
    (346, 256, 1024, 0, 0, 1), (1024, 256, 346, 1, 0, 1), (346, 1024, 256, 0, 1, 1), (512, 128, 6844, 1, 0, 64),
    (200, 72, 104, 0, 0, 1), (200, 72, 104, 1, 1, 1), (36, 8, 12, 1, 0, 1)])
def test_gemm_against_float64(rows, cols, inner, at, bt, split):
    from pccnn_lib_amd import _lib
    rng = np.random.default_rng(rows + cols + inner)
    a = rng.normal(size=(inner, rows) if at else (rows, inner)).astype(np.float32)
    b = rng.normal(size=(cols, inner) if bt else (inner, cols)).astype(np.float32)
    ta, tb = t(a), t(b)
    tc = torch.full((rows, cols), float("nan"), dtype=torch.float32, device=DEV)
    ws = torch.empty(split * rows * cols * 4 + 256, dtype=torch.uint8, device=DEV)
    _lib.call("pccnn_gemm_f32", _lib.P(ta.data_ptr()), _lib.P(tb.data_ptr()), _lib.P(tc.data_ptr()), rows, cols, inner,
              at, bt, a.shape[1], b.shape[1], cols, 1, 0, 0, 0, split, _lib.P(ws.data_ptr()), ws.numel(),
              _lib.P(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    exp = (a.T if at else a).astype(np.float64) @ (b.T if bt else b).astype(np.float64)
    assert relerr(tc.cpu().numpy(), exp) < 1e-5


@pytest.mark.parametrize("m,mlps,inner,co", [(200, 2, 48, 24), (256, 2, 208, 128), (32768, 3, 192, 128)])
def test_gemm_batched_strided(m, mlps, inner, co):
    # the second and third shapes have full tiles: the kernel without bounds checks, 64-row and 128-row tiles
    from pccnn_lib_amd import _lib
    rng = np.random.default_rng(0)
    a = rng.normal(size=(m, mlps * inner)).astype(np.float32)
    b = rng.normal(size=(mlps, inner, co)).astype(np.float32)
    ta, tb = t(a), t(b)
    tc = torch.zeros((m, mlps * co), dtype=torch.float32, device=DEV)
    _lib.call("pccnn_gemm_f32", _lib.P(ta.data_ptr()), _lib.P(tb.data_ptr()), _lib.P(tc.data_ptr()), m, co, inner, 0, 0,
              mlps * inner, co, mlps * co, mlps, inner, inner * co, co, 1, _lib.P(0), 0,
              _lib.P(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    exp = np.concatenate([a[:, i * inner:(i + 1) * inner].astype(np.float64) @ b[i] for i in range(mlps)], axis=1)
    assert relerr(tc.cpu().numpy(), exp) < 1e-5


# ------------------------------------------------------------------------------------- pdf

@pytest.mark.parametrize("bw", [0.025, 0.01, 0.1])
def test_pdf_matches_oracle(ops, oracle, models, bw):
    # bw = 0.1 reaches the 300-neighbor cap (deterministic subset, same in the oracle's restatement)
    pts, ids = _cloud(models, 4, 1000)
    exp_unnorm, exp_norm, exp_nb = oracle.pointcloud_pdf(pts, ids, bw)
    import pccnn_lib_amd as lib
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pc.compute_pdf(np.full(3, bw, np.float32))
    torch.cuda.synchronize()
    assert relerr(pc.pts_unnorm_pdf_.cpu().numpy(), exp_unnorm) < FWD_TOL
    assert relerr(pc.pts_pdf_.cpu().numpy(), exp_norm) < FWD_TOL
    assert np.allclose(pc.pts_unnorm_pdf_.cpu().numpy(), exp_unnorm, rtol=1e-5, atol=0)


@pytest.mark.parametrize("cap", [0, 300, 7])
def test_pdf_from_the_grid_equals_the_list_route(ops, models, cap):
    """compute_pdf_grid sums what compute_pdf sums over the (capped) neighbor list of the same grid, in the same
    order: with double accumulation the two agree to the last bit or two of the fp32 result."""
    import pccnn_lib_amd as lib
    pts, ids = _cloud(models, 3, 1000)
    rooms = (synthetic.room(11, 20000) / 10.0).astype(np.float32)
    large = synthetic.room(12, 150000)                    # one point per lane; the smaller clouds run 8 lanes per point
    for cloud, cloud_ids, bw in ((pts, ids, 0.05), (rooms, np.zeros(rooms.shape[0], np.int32), 0.004),
                                 (large, np.zeros(large.shape[0], np.int32), 0.012)):
        pc = lib.pc.Pointcloud(cloud, cloud_ids, device=DEV)
        bandwidth = torch.full((3,), bw, device=DEV)
        grid = lib.pc.Grid(pc, lib.pc.BoundingBox(pc), bandwidth * 4.0)
        grid.compute_cell_ids()
        grid.build_ds()
        neigh, ends = ops.find_neighbors_ex(grid.sorted_pts_, grid.sorted_cell_ids_, grid.sorted_pts_,
                                            grid.sorted_cell_ids_, grid.grid_ds_, grid.num_cells_, grid.cell_size_, cap,
                                            sample_order=grid.sorted_ids_i32_, cell_table=grid.cell_table_,
                                            samples_presorted=True)
        want = ops.compute_pdf_sorted(3, bandwidth, grid.sorted_pts_, pc.pts_, neigh, ends)
        per_cloud = pc.get_num_points_per_batch().to(torch.float32)[pc.batch_ids_.to(torch.int64)]
        for table in (grid.cell_table_, None):
            got, normed = ops.compute_pdf_grid(3, bandwidth, grid.sorted_pts_, grid.sorted_cell_ids_,
                                               grid.sorted_ids_i32_, grid.grid_ds_, grid.num_cells_, grid.cell_size_,
                                               cap, cell_table=table, with_normalized=True)
            torch.cuda.synchronize()
            assert np.allclose(got.cpu().numpy(), want.cpu().numpy(), rtol=3e-7, atol=0)
            assert torch.equal(normed, got / per_cloud)        # the cloud's point count, found from the sorted keys
        if cap == 7:
            counts = np.diff(np.concatenate([[0], ends.cpu().numpy()]))
            assert counts.max() == 7                          # the cap is reached, the subset rule is exercised
        # points already in key order, no sample_order: the result comes out in that order
        direct = ops.compute_pdf_grid(3, bandwidth, grid.sorted_pts_, grid.sorted_cell_ids_, None, grid.grid_ds_,
                                      grid.num_cells_, grid.cell_size_, cap, cell_table=grid.cell_table_)
        assert torch.equal(direct, got[grid.sorted_ids_.to(torch.int64)])


def test_pdf_grads_match_oracle(ops, oracle, models):
    pts, ids = _cloud(models, 2, 500)
    bw = np.full(3, 0.08, np.float32)
    _, _, nb = oracle.pointcloud_pdf(pts, ids, bw)
    g = np.random.default_rng(0).normal(size=pts.shape[0]).astype(np.float32)
    exp = oracle.compute_pdf_grads(3, bw, pts, nb["neighbors"], nb["ends"], g)
    got = ops.compute_pdf_grads(3, t(bw), t(pts), t(nb["neighbors"]), t(nb["ends"]), t(g))
    assert relerr(got.cpu().numpy(), exp) < GRAD_TOL
    # through autograd: d mean(pdf) / d pts
    import pccnn_lib_amd as lib
    pc = lib.pc.Pointcloud(pts, ids, device=DEV, requires_grad=True)
    pc.compute_pdf(bw)
    pc.pts_unnorm_pdf_.mean().backward()
    exp2 = oracle.compute_pdf_grads(3, bw, pts, nb["neighbors"], nb["ends"],
                                    np.full(pts.shape[0], 1.0 / pts.shape[0], np.float32))
    assert relerr(pc.pts_.grad.cpu().numpy(), exp2) < GRAD_TOL


# ------------------------------------------------------------------------------------ conv

def _conv_case(oracle, ops, seed, batch, num_pts, radius, distinct_samples):
    pts, ids = synthetic.primitives(seed, batch, num_pts)
    rng = np.random.default_rng(seed)
    if distinct_samples:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    nb = gpu_neighborhood(ops, pts, ids, smp, sids, radius, batch)
    return pts, ids, smp, nb, rng


@pytest.mark.parametrize("k,c_in,c_out,distinct", [(15, 32, 32, False), (16, 64, 48, True), (8, 5, 7, True),
                                                   (33, 128, 16, False), (64, 16, 8, True)])
def test_kpconv_forward_and_grads(ops, oracle, k, c_in, c_out, distinct):
    pts, ids, smp, nb, rng = _conv_case(oracle, ops, 20 + k, 2, 1500, 0.12, distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    d = nb["dev"]
    out = ops.kp_conv(d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    exp = oracle.kpconv(pts, feats, smp, neigh, ends, radii, kp, sigma, w)
    assert relerr(out.cpu().numpy(), exp) < FWD_TOL
    grads = ops.kp_conv_grads(d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w),
                              t(g))
    exp_g = oracle.kpconv_grads(pts, feats, smp, neigh, ends, radii, kp, sigma, w, g)
    for got, e, name in zip(grads, exp_g, ("dW", "dFeat", "dKernelPts", "dPts", "dSamples")):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < GRAD_TOL, name
        assert mixed_close(got.cpu().numpy(), e), name


@pytest.mark.parametrize("hidden,mlps,c_in,c_out,distinct", [(16, 1, 64, 128, False), (8, 2, 32, 24, True),
                                                             (16, 1, 3, 16, True), (4, 4, 8, 8, False)])
def test_mcconv_forward_and_grads(ops, oracle, hidden, mlps, c_in, c_out, distinct):
    pts, ids, smp, nb, rng = _conv_case(oracle, ops, 40 + hidden + mlps, 2, 1500, 0.12, distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    k = hidden * mlps
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, k)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, k)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * hidden)), (mlps, hidden * c_in, c_out // mlps)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    d = nb["dev"]
    args = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(w))
    out = ops.mc_conv(*args)
    exp = oracle.mcconv(pts, pdf, feats, smp, neigh, ends, radii, axis, bias, w)
    assert relerr(out.cpu().numpy(), exp) < FWD_TOL
    grads = ops.mc_conv_grads(*args, t(g))
    exp_g = oracle.mcconv_grads(pts, pdf, feats, smp, neigh, ends, radii, axis, bias, w, g)
    for got, e, name in zip(grads, exp_g, ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < GRAD_TOL, name
        assert mixed_close(got.cpu().numpy(), e), name


def test_config1_plumbing_kpconv_layer(oracle):
    # 2 x 1024 sphere points, radius 0.1, K = 15, sigma 0.05, 32 -> 32: through the layer API
    import pccnn_lib_amd as lib
    pts = np.concatenate([synthetic.sphere_surface(np.random.default_rng(s), 1024) for s in (0, 1)])
    ids = np.repeat(np.arange(2, dtype=np.int32), 1024)
    rng = np.random.default_rng(2)
    feats = rng.normal(size=(2048, 32)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (15 * 32)), (15 * 32, 32)).astype(np.float32)
    for sigma in (0.05, None):
        torch.manual_seed(0)
        layer = lib.pc.layers.KPConv(3, 32, 32, 15).to(DEV)
        layer.conv_weights_.data.copy_(t(w))
        if sigma is not None:
            layer.sigma_.fill_(sigma)
        pc = lib.pc.Pointcloud(pts, ids, device=DEV)
        out, nbh = layer(pc, pc, t(feats), 0.1)
        exp_nb = oracle.neighborhood(pts, ids, pts, ids, 0.1)
        assert np.array_equal(oracle.canonical_pairs(nbh.neighbors_.cpu().numpy()),
                              oracle.canonical_pairs(exp_nb["neighbors"]))
        exp = oracle.kpconv(pts, feats, pts, exp_nb["neighbors"], exp_nb["ends"], exp_nb["radii"],
                            layer.kernel_pts_.cpu().numpy(), float(layer.sigma_.item()), w)
        assert relerr(out.detach().cpu().numpy(), exp) < FWD_TOL


def test_mcconv_layer_autograd_routing(oracle):
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(9, 2, 1200)
    rng = np.random.default_rng(3)
    feats = rng.normal(size=(pts.shape[0], 16)).astype(np.float32)
    torch.manual_seed(1)
    layer = lib.pc.layers.MCConv(3, 16, 32, 16).to(DEV)
    layer.proj_bias_.data.normal_(0, 0.1)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pc.compute_pdf(np.full(3, 0.02, np.float32))
    tf = t(feats).requires_grad_(True)
    out, nbh = layer(pc, pc, tf, 0.1)
    g = rng.normal(size=tuple(out.shape)).astype(np.float32)
    out.backward(t(g))
    nb = dict(neighbors=nbh.neighbors_.cpu().numpy(), ends=nbh.start_ids_.cpu().numpy())
    radii = np.full(3, 0.1, np.float32)
    pdf = (pc.pts_unnorm_pdf_ * torch.prod(t(radii))).cpu().numpy()
    p = lambda x: x.detach().cpu().numpy()
    exp_g = oracle.mcconv_grads(pts, pdf, feats, pts, nb["neighbors"], nb["ends"], radii, p(layer.proj_axis_),
                                p(layer.proj_bias_), p(layer.conv_weights_), g)
    assert relerr(p(layer.conv_weights_.grad), exp_g[0]) < GRAD_TOL
    assert relerr(p(tf.grad), exp_g[1]) < GRAD_TOL
    assert relerr(p(layer.proj_axis_.grad), exp_g[2]) < GRAD_TOL
    assert relerr(p(layer.proj_bias_.grad), exp_g[3]) < GRAD_TOL


def test_point_gradient_through_density_and_mcconv_equals_the_composed_oracle(oracle):
    # unit_test/test_mcconv_pt_grads.py:92-103: points -> Pointcloud.compute_pdf -> pdf * prod(radius) -> MCConv with
    # the same tensor as points and samples; pts.grad = dPts + dSamples + compute_pdf_grads(dPdf * prod(radius)).
    # The three terms come from two different ops and are added by autograd; here the sum is compared with the
    # oracle's mcconv_grads and compute_pdf_grads composed by hand (3-D, full kernels).
    import pccnn_lib_amd as lib
    from pccnn_lib_amd.op_wrappers import ComputeMCConv
    pts, ids = synthetic.primitives(17, 2, 1200)
    rng = np.random.default_rng(17)
    c_in, c_out, hidden, radius = 16, 24, 8, 0.1
    bw = np.full(3, 0.025, np.float32)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, hidden)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * hidden)), (1, hidden * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    radii = np.full(3, radius, np.float32)

    pc = lib.pc.Pointcloud(pts, ids, device=DEV, requires_grad=True)
    pc.compute_pdf(bw)
    assert pc.pts_unnorm_pdf_.requires_grad
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, t(radii), 0)
    cur_pdf = pc.pts_unnorm_pdf_ * torch.prod(t(radii))
    out = ComputeMCConv.apply(pc.pts_, cur_pdf, t(feats), pc.pts_, nbh.neighbors_, nbh.start_ids_, t(radii), t(axis),
                              t(bias), t(w))
    (out * t(g)).sum().backward()
    got = pc.pts_.grad.cpu().numpy()

    unnorm, _, nb_pdf = oracle.pointcloud_pdf(pts, ids, bw)
    nb = oracle.neighborhood(pts, ids, pts, ids, radius)
    pdf = (unnorm * np.prod(radii)).astype(np.float32)
    assert relerr(cur_pdf.detach().cpu().numpy(), pdf) < FWD_TOL
    eg = oracle.mcconv_grads(pts, pdf, feats, pts, nb["neighbors"], nb["ends"], radii, axis, bias, w, g)
    through_pdf = oracle.compute_pdf_grads(3, bw, pts, nb_pdf["neighbors"], nb_pdf["ends"],
                                           (eg[4] * np.prod(radii)).astype(np.float32))
    direct = eg[5] + eg[6]
    exp = direct + through_pdf
    # both routes carry weight: neither term alone satisfies the tolerance
    assert relerr(direct, exp) > 100 * GRAD_TOL and relerr(through_pdf, exp) > 100 * GRAD_TOL
    assert relerr(got, exp) < GRAD_TOL
    assert mixed_close(got, exp)


def test_hierarchy_level_with_pooling(oracle):
    # one level of a hierarchical encoder: Poisson-disk pooling, then an MCConv from the fine cloud to the pooled one
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(13, 2, 3000)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pool = lib.pc.PointPooling(pc, torch.full((3,), 0.05, device=DEV))
    sel = pool.pooling_ids_.cpu().numpy()
    pooled_pts, pooled_ids = pts[sel], ids[sel]
    for b in range(2):
        q = pooled_pts[pooled_ids == b].astype(np.float64)
        dist = np.linalg.norm(q[:, None] - q[None], axis=-1) + np.eye(q.shape[0]) * 1e9
        assert dist.min() >= 0.05 * (1 - 1e-6)
    pc_out = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
    pc.compute_pdf(np.full(3, 0.01, np.float32))
    rng = np.random.default_rng(5)
    feats = rng.normal(size=(pts.shape[0], 8)).astype(np.float32)
    torch.manual_seed(2)
    layer = lib.pc.layers.MCConv(3, 8, 16, 16).to(DEV)
    out, nbh = layer(pc, pc_out, t(feats), 0.1)
    exp_nb = oracle.neighborhood(pts, ids, pooled_pts, pooled_ids, 0.1)
    assert np.array_equal(oracle.canonical_pairs(nbh.neighbors_.cpu().numpy()),
                          oracle.canonical_pairs(exp_nb["neighbors"]))
    p = lambda x: x.detach().cpu().numpy()
    pdf = p(pc.pts_unnorm_pdf_ * 0.1 ** 3)
    exp = oracle.mcconv(pts, pdf, feats, pooled_pts, exp_nb["neighbors"], exp_nb["ends"], exp_nb["radii"],
                        p(layer.proj_axis_), p(layer.proj_bias_), p(layer.conv_weights_))
    assert relerr(p(out), exp) < 2e-5


def test_cached_projection_and_gradient_masks(ops, oracle):
    # the projection kept from the forward call gives the same gradients as rebuilding it, and a gradient
    # mask returns exactly the requested groups (the others are None), each equal to the full call's
    pts, ids, smp, nb, rng = _conv_case(oracle, ops, 91, 2, 1200, 0.12, True)
    d = nb["dev"]
    c_in, c_out, k = 32, 16, 16
    feats = t(rng.normal(size=(pts.shape[0], c_in)).astype(np.float32))
    pdf = t(rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32))
    axis = t(rng.normal(0, 0.6, (3, k)).astype(np.float32))
    bias = t(rng.normal(0, 0.1, (1, k)).astype(np.float32))
    w = t(rng.normal(0, 0.1, (1, k * c_in, c_out)).astype(np.float32))
    g = t(rng.normal(size=(smp.shape[0], c_out)).astype(np.float32))
    args = (d["pts"], pdf, feats, d["samples"], d["neigh"], d["ends"], d["radii"], axis, bias, w)
    out, proj = ops.mc_conv(*args, return_proj=True)
    assert tuple(proj.shape) == (smp.shape[0], c_in, k) and torch.equal(out, ops.mc_conv(*args))
    full = ops.mc_conv_grads(*args, g)
    cached = ops.mc_conv_grads(*args, g, proj=proj)
    for a, b in zip(full, cached):
        assert relerr(a.cpu().numpy(), b.cpu().numpy()) < 1e-6
    fw = ops.mc_conv_grads(*args, g, proj=proj, grad_mask=ops.GRAD_WEIGHTS | ops.GRAD_FEATS)
    assert [x is None for x in fw] == [False, False, True, True, True, True, True]
    assert torch.equal(fw[0], cached[0]) and relerr(fw[1].cpu().numpy(), full[1].cpu().numpy()) < 1e-6
    par = ops.mc_conv_grads(*args, g, grad_mask=ops.GRAD_BASIS_PARAMS | ops.GRAD_PDF)
    assert [x is None for x in par] == [True, True, False, False, False, True, True]
    assert relerr(par[2].cpu().numpy(), full[2].cpu().numpy()) < 1e-6
    assert relerr(par[4].cpu().numpy(), full[4].cpu().numpy()) < 1e-5
    ptsg = ops.mc_conv_grads(*args, g, grad_mask=ops.GRAD_PTS)
    assert relerr(ptsg[5].cpu().numpy(), full[5].cpu().numpy()) < 1e-5
    assert relerr(ptsg[6].cpu().numpy(), full[6].cpu().numpy()) < 1e-6
    # autograd asks only for what requires grad
    from pccnn_lib_amd.op_wrappers import ComputeMCConv
    wr = w.clone().requires_grad_(True)
    fr = feats.clone().requires_grad_(True)
    res = ComputeMCConv.apply(d["pts"], pdf, fr, d["samples"], d["neigh"], d["ends"], d["radii"], axis, bias, wr)
    gw, gf = torch.autograd.grad(res, [wr, fr], g)
    assert torch.equal(gw, cached[0]) and relerr(gf.cpu().numpy(), full[1].cpu().numpy()) < 1e-6


@pytest.mark.parametrize("c_in", [8, 32, 64])
def test_parameter_gradients_alone_equal_the_full_call(ops, oracle, c_in):
    # with no gradient towards positions, samples or densities asked for, the backward projection leaves out the
    # per-pair geometry sums; the features' and the basis parameters' gradients are those of the full call
    pts, ids, smp, nb, rng = _conv_case(oracle, ops, 92, 2, 1500, 0.12, True)
    d = nb["dev"]
    c_out, k = 16, 8
    feats = t(rng.normal(size=(pts.shape[0], c_in)).astype(np.float32))
    pdf = t(rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32))
    axis = t(rng.normal(0, 0.6, (3, k)).astype(np.float32))
    bias = t(rng.normal(0, 0.1, (1, k)).astype(np.float32))
    w = t(rng.normal(0, 0.1, (1, k * c_in, c_out)).astype(np.float32))
    g = t(rng.normal(size=(smp.shape[0], c_out)).astype(np.float32))
    args = (d["pts"], pdf, feats, d["samples"], d["neigh"], d["ends"], d["radii"], axis, bias, w)
    full = ops.mc_conv_grads(*args, g)
    for mask in (ops.GRAD_BASIS_PARAMS, ops.GRAD_BASIS_PARAMS | ops.GRAD_FEATS | ops.GRAD_WEIGHTS):
        some = ops.mc_conv_grads(*args, g, grad_mask=mask)
        assert some[4] is None and some[5] is None and some[6] is None       # density, positions, samples
        assert relerr(some[2].cpu().numpy(), full[2].cpu().numpy()) < 1e-5      # axes
        assert relerr(some[3].cpu().numpy(), full[3].cpu().numpy()) < 1e-5      # biases
        if mask & ops.GRAD_FEATS:
            assert relerr(some[1].cpu().numpy(), full[1].cpu().numpy()) < 1e-6


def test_weight_variance_ops_and_layer_warmup(ops, oracle):
    import pccnn_lib_amd as lib
    pts, ids, smp, nb, rng = _conv_case(oracle, ops, 77, 2, 1500, 0.12, True)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    d = nb["dev"]
    feats = rng.normal(size=(pts.shape[0], 24)).astype(np.float32)
    kp, sigma = synthetic.kernel_points_sphere(1, 15)
    got = ops.kp_conv_weight_var(d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma)
    assert got.dim() == 0
    exp = oracle.kpconv_weight_var(pts, feats, smp, neigh, ends, radii, kp, sigma)
    assert abs(float(got) - float(exp)) < 1e-5 * abs(float(exp))
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    axis = rng.normal(0, 0.6, (3, 16)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, 16)).astype(np.float32)
    got = ops.mc_conv_weight_var(d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis),
                                 t(bias))
    exp = oracle.mcconv_weight_var(pts, pdf, feats, smp, neigh, ends, radii, axis, bias)
    assert abs(float(got) - float(exp)) < 1e-5 * abs(float(exp))
    # the layers' warm-up path (KPConv.py:103-116): weights are redrawn with the variance the statistic asks for
    torch.manual_seed(3)
    layer = lib.pc.layers.KPConv(3, 24, 8, 15, True, 1.0).to(DEV)
    layer.set_init_warmup_state(True)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    out, nbh = layer(pc, pc, t(feats), 0.12)
    var = oracle.kpconv_weight_var(pts, feats, pts, nbh.neighbors_.cpu().numpy(), nbh.start_ids_.cpu().numpy(),
                                   np.full(3, 0.12, np.float32), layer.kernel_pts_.cpu().numpy(), layer.sigma_cpu_)
    assert abs(layer.accum_weight_var_ - 1.0 / float(var)) < 1e-4 * abs(1.0 / float(var))
    # with weights of that variance the output variance is about the requested constant
    assert 0.5 < float(out.detach().var()) < 2.0


def test_model_base_class_runs_the_warmup_of_its_layers(ops, oracle):
    # the loop a trainer built on the reference runs (IModel.py:19-27 with KPConv.py:103-116): layer after layer is
    # switched into its warm-up state, fed a batch so that it measures its statistic and redraws its weights, and
    # switched back; afterwards every layer's output variance is about the constant asked for
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(5, 2, 2000)
    rng = np.random.default_rng(5)
    feats = t(rng.normal(size=(pts.shape[0], 16)).astype(np.float32))
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pc.compute_pdf(np.full(3, 0.02, np.float32))
    torch.manual_seed(11)
    model = lib.pc.models.IModel()
    model.add_conv(lib.pc.layers.KPConv(3, 16, 32, 15, True, 1.0).to(DEV))
    model.add_conv(lib.pc.layers.MCConv(3, 32, 32, 8, 1, True, 1.0).to(DEV))
    assert model.get_num_convs() == 2

    def forward():
        first, nbh = model.conv_list_[0](pc, pc, feats, 0.12)
        return first, model.conv_list_[1](pc, pc, torch.nn.functional.leaky_relu(first, 0.2), 0.12, nbh)

    with torch.no_grad():
        for i in range(model.get_num_convs()):
            model.init_variance(i, 1.0)
            model.set_init_warmup_state(i, True)
            forward()
            model.set_init_warmup_state(i, False)
            assert model.conv_list_[i].accum_weight_var_ > 0.0
        mid, out = forward()
    assert 0.5 < float(mid.var()) < 2.0 and 0.5 < float(out.var()) < 2.0   # (measured: 0.94 - 1.05)


def test_error_paths(ops):
    pts, ids = synthetic.primitives(1, 1, 128)
    tp, ti = t(pts), t(ids)
    with pytest.raises(RuntimeError, match="dtype"):
        ops.compute_keys(tp, ti.to(torch.int64), tp[:1], torch.ones(3, dtype=torch.int32, device=DEV), tp[0])
    with pytest.raises(RuntimeError, match="not supported"):
        ops.bounding_box(tp[:, :1].contiguous(), ti, 1)
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.bounding_box(tp.t().contiguous().t(), ti, 1)
    nb = gpu_neighborhood(ops, pts, ids, pts, ids, 0.2, 1)["dev"]
    feats = torch.zeros((128, 4), device=DEV)
    with pytest.raises(RuntimeError, match="k=65"):
        ops.kp_conv(tp, feats, tp, nb["neigh"], nb["ends"], nb["radii"], torch.zeros((65, 3), device=DEV), 0.3,
                    torch.zeros((65 * 4, 2), device=DEV))


def test_mirror_index_and_atomic_free_point_gradients(ops, oracle):
    # samples == points, uncapped search: the pair list is symmetric, its mirror index exists, and the backward
    # pass that gathers per point with it gives the gradients of the atomic path and of the oracle
    pts, ids, smp, nb, rng = _conv_case(oracle, ops, 77, 2, 1500, 0.12, False)
    d = nb["dev"]
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    mirror = ops.mirror_pairs(d["neigh"], d["ends"])
    assert mirror is not None
    mi = mirror.cpu().numpy()
    assert np.array_equal(mi[mi], np.arange(mi.shape[0]))
    assert np.array_equal(neigh[mi], neigh[:, ::-1])
    k, c_in, c_out = 16, 32, 24
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    g = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, k)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, k)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * k)), (1, k * c_in, c_out)).astype(np.float32)
    args = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(w), t(g))
    atomic = ops.mc_conv_grads(*args)
    gathered = ops.mc_conv_grads(*args, mirror=mirror)
    exp = oracle.mcconv_grads(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, w, g)
    for a, b, e, name in zip(atomic, gathered, exp, ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")):
        assert relerr(b.cpu().numpy(), e) < GRAD_TOL, name
        assert relerr(b.cpu().numpy(), a.cpu().numpy()) < GRAD_TOL, name
    # the gather sums in a fixed order: two runs agree bit for bit
    again = ops.mc_conv_grads(*args, mirror=mirror)
    assert torch.equal(again[5], gathered[5]) and torch.equal(again[4], gathered[4])
    kp, sigma = synthetic.kernel_points_sphere(1, 15)
    wk = rng.normal(0, 0.1, (15 * c_in, c_out)).astype(np.float32)
    kargs = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(wk), t(g))
    got = ops.kp_conv_grads(*kargs, mirror=mirror)
    exp = oracle.kpconv_grads(pts, feats, pts, neigh, ends, radii, kp, sigma, wk, g)
    for b, e, name in zip(got, exp, ("dW", "dFeat", "dKernelPts", "dPts", "dSamples")):
        assert relerr(b.cpu().numpy(), e) < GRAD_TOL, name
    # a subset of the points as samples is not symmetric: no mirror index, and passing one is refused
    _, _, smp2, nb2, _ = _conv_case(oracle, ops, 78, 2, 900, 0.12, True)
    d2 = nb2["dev"]
    assert ops.mirror_pairs(d2["neigh"], d2["ends"]) is None
    with pytest.raises(RuntimeError, match="mirror"):
        ops.kp_conv_grads(d2["pts"], torch.zeros((d2["pts"].shape[0], c_in), device=DEV), d2["samples"], d2["neigh"],
                          d2["ends"], d2["radii"], t(kp), sigma, t(wk),
                          torch.zeros((d2["samples"].shape[0], c_out), device=DEV),
                          mirror=torch.zeros(d2["neigh"].shape[0], dtype=torch.int32, device=DEV))


def test_layer_uses_mirror_for_point_gradients(oracle):
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(21, 2, 1000)
    rng = np.random.default_rng(21)
    feats = rng.normal(size=(pts.shape[0], 8)).astype(np.float32)
    torch.manual_seed(7)
    layer = lib.pc.layers.KPConv(3, 8, 12, 15).to(DEV)
    tp = t(pts).requires_grad_(True)
    pc = lib.pc.Pointcloud(tp, ids, device=DEV)
    out, nbh = layer(pc, pc, t(feats), 0.1)
    assert nbh.mirror_ is not False and nbh.mirror_ is not None          # computed because the points need gradients
    g = rng.normal(size=tuple(out.shape)).astype(np.float32)
    out.backward(t(g))
    exp = oracle.kpconv_grads(pts, feats, pts, nbh.neighbors_.cpu().numpy(), nbh.start_ids_.cpu().numpy(),
                              np.full(3, 0.1, np.float32), layer.kernel_pts_.cpu().numpy(), float(layer.sigma_.item()),
                              layer.conv_weights_.detach().cpu().numpy(), g)
    assert relerr(tp.grad.cpu().numpy(), exp[3] + exp[4]) < GRAD_TOL


def test_ops_run_on_torch_current_stream(ops, models):
    # the native calls take torch's current stream: inside a stream context that is the side stream, and inputs
    # produced there by a slow producer are consumed in order without any device-wide synchronisation
    import pccnn_lib_amd as lib
    pts, ids = _cloud(models, 2, 1000)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    radii = torch.full((3,), 0.1, device=DEV)
    rng = np.random.default_rng(12)
    feats = t(rng.normal(size=(pts.shape[0], 16)).astype(np.float32))
    kpts = t(rng.normal(0, 0.5, (15, 3)).astype(np.float32))
    w = t(rng.normal(0, 0.2, (15 * 16, 8)).astype(np.float32))
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    want = ops.kp_conv(pc.pts_, feats, pc.pts_, nbh.neighbors_, nbh.start_ids_, radii, kpts, 0.3, w)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    assert (ops._stream().value or 0) == torch.cuda.current_stream().cuda_stream
    with torch.cuda.stream(side):
        assert (ops._stream().value or 0) == side.cuda_stream
        big = torch.randn((6144, 6144), device=DEV)
        feats_side = feats + (big @ big).sum() * 0.0          # ready only after a few milliseconds of side-stream work
        nbh_side = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
        got = ops.kp_conv(pc.pts_, feats_side, pc.pts_, nbh_side.neighbors_, nbh_side.start_ids_, radii, kpts, 0.3, w)
    side.synchronize()
    assert torch.equal(nbh_side.neighbors_, nbh.neighbors_)
    assert torch.equal(got, want)
    torch.cuda.synchronize()


def test_density_times_volume_on_the_host_equals_the_device_product():
    # an isotropic radius given as a host value: prod(radius) is taken on the host in fp32 and multiplies the densities
    # as a scalar; it must be the number the device reduction gives, bit for bit, for any radius
    from pccnn_lib_amd.pc._consts import device_vector, host_vector
    from pccnn_lib_amd.pc.layers.conv_base import density_times_volume
    rng = np.random.default_rng(3)
    pdf = t(rng.uniform(0.0, 50.0, 4096).astype(np.float32))
    for r in [0.05, 0.1, 0.025, 0.4, 1.0, 3.0] + [float(v) for v in rng.uniform(1e-3, 10.0, 40)]:
        radius = device_vector(r, 3, DEV)
        assert host_vector(radius) is not None
        want = pdf * torch.prod(radius.clone())                # a tensor the host knows nothing about
        assert torch.equal(density_times_volume(pdf, radius), want)
    mixed = device_vector([0.1, 0.2, 0.05], 3, DEV)             # not isotropic: the device product as before
    assert torch.equal(density_times_volume(pdf, mixed), pdf * torch.prod(mixed))
