"""The compiled ``pccnn_lib_ops`` extension against the ctypes binding of the same C ABI: all 26 functions of
pccnn_lib_ops/ops_list.cpp:26-54 on the same inputs.  The rest of the GPU suite runs through the binding in use by
default (the compiled one when it has been built) and compares it with the oracle; here the two bindings are held
against each other, so that both are covered."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, relerr, t

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import build, pccnn_lib_ops
    import os
    if not os.path.exists(build.extension_path()):
        pytest.skip("the compiled extension has not been built")
    before = pccnn_lib_ops.use_binding("compiled")
    pccnn_lib_ops.use_binding(before)
    return pccnn_lib_ops


def _same(a, b, exact=True):
    if isinstance(a, (list, tuple)):
        assert isinstance(b, (list, tuple)) and len(a) == len(b)
        for x, y in zip(a, b):
            _same(x, y, exact)
        return
    if a is None or b is None:
        assert a is None and b is None
        return
    assert a.dtype == b.dtype and tuple(a.shape) == tuple(b.shape) and a.device == b.device
    if exact:
        assert torch.equal(a, b)
    else:       # sums that the kernels add up with float atomics: equal up to the order of the additions
        assert relerr(a.float().cpu().numpy(), b.float().cpu().numpy()) < 1e-5


def _both(ops, name, *args, exact=True, **kwargs):
    got = {which: ops.BINDINGS[which][name](*args, **kwargs) for which in ("ctypes", "compiled")}
    _same(got["ctypes"], got["compiled"], exact)
    return got["compiled"]


@pytest.mark.parametrize("dims,num_pts", [(3, 1500), (3, 6000), (2, 1500), (4, 700)])
def test_index_ops_agree(ops, dims, num_pts):
    rng = np.random.default_rng(dims + num_pts)
    if dims == 3:
        pts, ids = synthetic.primitives(3 + num_pts, 2, num_pts)
    else:
        pts = rng.random((2 * num_pts, dims), dtype=np.float32)
        ids = np.repeat(np.arange(2, dtype=np.int32), num_pts)
    radius = {2: 0.06, 3: 0.1, 4: 0.3}[dims]
    nb = gpu_neighborhood(ops, pts, ids, pts, ids, radius, 2)
    d = nb["dev"]
    keys = _both(ops, "compute_keys", d["pts"], d["ids"], t(nb["aabb_min"]), d["nc"], d["radii"])
    assert np.array_equal(keys.cpu().numpy(), nb["keys"])
    shape = [2] + nb["num_cells"].tolist()[0:2] + [2]
    _both(ops, "build_grid_ds", d["skeys"], d["nc"], shape)
    # more than 4096 samples take the route that walks the samples in cell order; fewer take the plain one
    for cap in (0, 5):
        neigh, ends = _both(ops, "find_neighbors", d["spts"], d["skeys"], d["pts"], keys, d["ds"], d["nc"], d["radii"], cap)
    neigh, ends = _both(ops, "find_neighbors", d["spts"], d["skeys"], d["spts"], d["skeys"], d["ds"], d["nc"],
                        d["radii"], 0)
    sel = _both(ops, "poisson_disk_sampling", d["skeys"], neigh, ends, d["nc"])
    assert sel.shape[0] > 0
    bw = torch.full((dims,), 0.5 * radius, device=DEV)
    pdf = _both(ops, "compute_pdf", dims, bw, d["pts"], d["neigh"], d["ends"])
    assert float(pdf.min()) > 0
    g = t(rng.normal(size=pts.shape[0]).astype(np.float32))
    _both(ops, "compute_pdf_grads", dims, bw, d["pts"], d["neigh"], d["ends"], g, exact=False)
    empty = ops.BINDINGS["compiled"]["find_neighbors"](d["spts"], d["skeys"], d["pts"][:0], keys[:0], d["ds"], d["nc"],
                                                       d["radii"], 0)
    assert tuple(empty[0].shape) == (0, 2) and tuple(empty[1].shape) == (0,)


def _conv_inputs(ops, dims, seed, distinct):
    rng = np.random.default_rng(seed)
    if dims == 3:
        pts, ids = synthetic.primitives(seed, 2, 1200)
    else:
        pts = rng.random((2400, dims), dtype=np.float32)
        ids = np.repeat(np.arange(2, dtype=np.int32), 1200)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    nb = gpu_neighborhood(ops, pts, ids, smp, sids, {2: 0.06, 3: 0.12, 4: 0.3}[dims], 2)
    return nb["dev"], rng


@pytest.mark.parametrize("dims,distinct", [(3, False), (3, True), (2, False), (4, True)])
def test_kernel_point_families_agree(ops, dims, distinct):
    d, rng = _conv_inputs(ops, dims, 50 + dims, distinct)
    n, m = d["pts"].shape[0], d["samples"].shape[0]
    c_in, c_out, k = 16, 24, 15
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    kp = kp[:, :dims] if dims < 3 else np.concatenate([kp, kp[:, :dims - 3]], axis=1)
    kp = t(np.ascontiguousarray(kp, np.float32))
    feats = t(rng.normal(size=(n, c_in)).astype(np.float32))
    pdf = t(rng.uniform(0.5, 2.0, n).astype(np.float32))
    w = t(rng.normal(0, 0.1, (k * c_in, c_out)).astype(np.float32))
    g = t(rng.normal(size=(m, c_out)).astype(np.float32))
    geo = (d["samples"], d["neigh"], d["ends"], d["radii"])
    mirror = None if distinct or dims != 3 else ops.mirror_pairs(d["neigh"], d["ends"])
    # KPConv, incl. the keyword additions
    out, proj = _both(ops, "kp_conv", d["pts"], feats, *geo, kp, sigma, w, return_proj=True)
    _same(out, _both(ops, "kp_conv", d["pts"], feats, *geo, kp, sigma, w))
    _both(ops, "kp_conv_grads", d["pts"], feats, *geo, kp, sigma, w, g, exact=False)
    part = _both(ops, "kp_conv_grads", d["pts"], feats, *geo, kp, sigma, w, g, proj=proj,
                 grad_mask=ops.GRAD_WEIGHTS | ops.GRAD_PTS, mirror=mirror, exact=mirror is not None)
    assert part[1] is None and part[2] is None and part[0] is not None and part[3] is not None
    _both(ops, "kp_conv_weight_var", d["pts"], feats, *geo, kp, sigma)
    if dims == 3:
        o16, p16 = _both(ops, "kp_conv", d["pts"], feats, *geo, kp, sigma, w, return_proj=True, contraction="bf16")
        assert p16.dtype == torch.bfloat16
        _both(ops, "kp_conv_grads", d["pts"], feats, *geo, kp, sigma, w, g, proj=p16, contraction="bf16", exact=False)
    # KPConvN and PCCNN (feats before pdf)
    _both(ops, "kp_conv_n", d["pts"], pdf, feats, *geo, kp, sigma, w)
    _both(ops, "kp_conv_n_grads", d["pts"], pdf, feats, *geo, kp, sigma, w, g, exact=False)
    _both(ops, "kp_conv_n_weight_var", d["pts"], pdf, feats, *geo, kp, sigma)
    _both(ops, "pccnn", d["pts"], feats, pdf, *geo, kp, sigma, w)
    grads = _both(ops, "pccnn_grads", d["pts"], feats, pdf, *geo, kp, sigma, w, g, exact=False)
    assert len(grads) == 6 and tuple(grads[3].shape) == (n,)
    _both(ops, "pccnn_weight_variance", d["pts"], feats, pdf, *geo, kp, sigma)


@pytest.mark.parametrize("dims,distinct,mlps", [(3, False, 1), (3, True, 2), (2, True, 1), (4, False, 1)])
def test_mcconv_and_pointconv_agree(ops, dims, distinct, mlps):
    d, rng = _conv_inputs(ops, dims, 60 + dims, distinct)
    n, m = d["pts"].shape[0], d["samples"].shape[0]
    c_in, c_out, hidden = 16, 24, 8
    k = hidden * mlps
    feats = t(rng.normal(size=(n, c_in)).astype(np.float32))
    pdf = t(rng.uniform(0.5, 2.0, n).astype(np.float32))
    axis = t(rng.normal(0, 0.6, (dims, k)).astype(np.float32))
    bias = t(rng.normal(0, 0.1, (1, k)).astype(np.float32))
    w = t(rng.normal(0, 0.1, (mlps, hidden * c_in, c_out // mlps)).astype(np.float32))
    g = t(rng.normal(size=(m, c_out)).astype(np.float32))
    geo = (d["samples"], d["neigh"], d["ends"], d["radii"])
    out, proj = _both(ops, "mc_conv", d["pts"], pdf, feats, *geo, axis, bias, w, return_proj=True)
    grads = _both(ops, "mc_conv_grads", d["pts"], pdf, feats, *geo, axis, bias, w, g, exact=False)
    assert len(grads) == 7 and tuple(grads[3].shape) == (1, k) and tuple(grads[2].shape) == (dims, k)
    part = _both(ops, "mc_conv_grads", d["pts"], pdf, feats, *geo, axis, bias, w, g, proj=proj,
                 grad_mask=ops.GRAD_WEIGHTS)
    assert all(x is None for x in part[1:]) and torch.equal(part[0], grads[0])
    _both(ops, "mc_conv_weight_var", d["pts"], pdf, feats, *geo, axis, bias)
    if dims == 3:
        _, p16 = _both(ops, "mc_conv", d["pts"], pdf, feats, *geo, axis, bias, w, return_proj=True, contraction="bf16")
        _both(ops, "mc_conv_grads", d["pts"], pdf, feats, *geo, axis, bias, w, g, proj=p16, contraction="bf16",
              exact=False)
    # PointConv: its basis op, the gradient of that, the convolution on a caller-given basis
    basis = _both(ops, "point_conv_basis", d["pts"], d["radii"], d["samples"], d["neigh"], axis, bias)
    assert tuple(basis.shape) == (d["neigh"].shape[0], k)
    gb = t(rng.normal(size=tuple(basis.shape)).astype(np.float32))
    _both(ops, "point_conv_basis_grads", d["pts"], d["radii"], d["samples"], d["neigh"], axis, bias, gb, exact=False)
    wp = t(rng.normal(0, 0.1, (k * c_in, c_out)).astype(np.float32))
    out, proj = _both(ops, "point_conv", basis, feats, d["neigh"], d["ends"], wp, return_proj=True)
    grads = _both(ops, "point_conv_grads", basis, feats, d["neigh"], d["ends"], wp, g, proj=proj, exact=False)
    assert len(grads) == 3 and tuple(grads[2].shape) == tuple(basis.shape)
    _both(ops, "point_conv_weight_var", basis, feats, d["neigh"], d["ends"])


def test_sphconv_agrees_and_rejects_other_dimensions(ops):
    d, rng = _conv_inputs(ops, 3, 71, True)
    n, m = d["pts"].shape[0], d["samples"].shape[0]
    c_in, c_out = 8, 12
    radial = t(np.array([0.0, 0.5], np.float32))
    azimuth = t(np.linspace(-np.pi, np.pi, 5)[:-1].astype(np.float32))
    polar = t(np.linspace(0.0, np.pi, 4)[:-1].astype(np.float32))
    k = 2 * 4 * 3 + 1
    feats = t(rng.normal(size=(n, c_in)).astype(np.float32))
    w = t(rng.normal(0, 0.1, (k * c_in, c_out)).astype(np.float32))
    g = t(rng.normal(size=(m, c_out)).astype(np.float32))
    geo = (d["samples"], d["neigh"], d["ends"], d["radii"])
    out, proj = _both(ops, "sph_conv", d["pts"], feats, *geo, radial, azimuth, polar, w, return_proj=True)
    grads = _both(ops, "sph_conv_grads", d["pts"], feats, *geo, radial, azimuth, polar, w, g, proj=proj, exact=False)
    assert len(grads) == 2
    _both(ops, "sph_conv_weight_var", d["pts"], feats, *geo, radial, azimuth, polar)
    d4, _ = _conv_inputs(ops, 4, 72, False)
    for which in ("ctypes", "compiled"):
        with pytest.raises(RuntimeError, match="3 only"):
            ops.BINDINGS[which]["sph_conv"](d4["pts"], feats[:d4["pts"].shape[0]], d4["samples"], d4["neigh"], d4["ends"],
                                            d4["radii"], radial, azimuth, polar, w)


@pytest.mark.parametrize("which", ["ctypes", "compiled"])
def test_contracts_are_checked_by_both_bindings(ops, which):
    f = ops.BINDINGS[which]
    pts = torch.rand(100, 3, device=DEV)
    ids = torch.zeros(100, dtype=torch.int32, device=DEV)
    mn = torch.zeros(1, 3, device=DEV)
    nc = torch.full((3,), 4, dtype=torch.int32, device=DEV)
    cell = torch.full((3,), 0.25, device=DEV)
    with pytest.raises(RuntimeError, match="dtype"):
        f["compute_keys"](pts, ids.to(torch.int64), mn, nc, cell)
    with pytest.raises(RuntimeError, match="contiguous"):
        f["compute_keys"](torch.rand(3, 100, device=DEV).t(), ids, mn, nc, cell)
    with pytest.raises(RuntimeError, match="inconsistent shapes"):
        f["compute_keys"](pts, ids[:50], mn, nc, cell)
    with pytest.raises(RuntimeError, match="out_shape"):
        f["build_grid_ds"](torch.zeros(100, dtype=torch.int64, device=DEV), nc, [1, 4, 4])
    with pytest.raises(RuntimeError, match="contraction"):
        f["kp_conv"](pts, pts, pts, torch.zeros(1, 2, dtype=torch.int32, device=DEV), ids, cell, pts[:15], 0.3,
                     torch.rand(45, 4, device=DEV), contraction="fp8")
