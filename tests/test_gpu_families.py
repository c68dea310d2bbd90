"""HIP path vs the CPU oracle for the convolution families beside KPConv / MCConv: KPConvN, PCCNN,
PointConv (basis op + convolution with explicit basis values) and SPHConv.  Same tolerances as the
KPConv / MCConv tests: outputs 1e-5 relative to the largest magnitude of the tensor, gradients 1e-4."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, relerr, t

pytestmark = pytest.mark.gpu

FWD_TOL = 1e-5
GRAD_TOL = 1e-4


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _case(ops, seed, distinct, num_pts=1500, radius=0.12):
    pts, ids = synthetic.primitives(seed, 2, num_pts)
    rng = np.random.default_rng(seed)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    nb = gpu_neighborhood(ops, pts, ids, smp, sids, radius, 2)
    return pts, smp, nb, rng


def _check(grads, expect, names):
    for got, e, name in zip(grads, expect, names):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < GRAD_TOL, name


@pytest.mark.parametrize("k,c_in,c_out,distinct", [(16, 32, 24, True), (15, 8, 5, False), (33, 64, 16, True)])
def test_kpconvn_forward_and_grads(ops, oracle, k, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 60 + k, distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    d = nb["dev"]
    args = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    out = ops.kp_conv_n(*args)
    assert relerr(out.cpu().numpy(), oracle.kpconvn(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma, w)) < FWD_TOL
    _check(ops.kp_conv_n_grads(*args, t(g)),
           oracle.kpconvn_grads(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma, w, g),
           ("dW", "dFeat", "dKernelPts", "dPts", "dSamples"))
    var = ops.kp_conv_n_weight_var(*args[:-1])
    exp = oracle.kpconvn_weight_var(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma)
    assert abs(float(var) - float(exp)) < 1e-5 * abs(float(exp))


@pytest.mark.parametrize("k,c_in,c_out,distinct", [(16, 32, 24, True), (8, 5, 7, False), (64, 16, 8, True)])
def test_pccnn_forward_and_grads(ops, oracle, k, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 80 + k, distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    kp, _ = synthetic.kernel_points_sphere(2, k)
    sigma = 0.35
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    d = nb["dev"]
    args = (d["pts"], t(feats), t(pdf), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    out = ops.pccnn(*args)
    assert relerr(out.cpu().numpy(), oracle.pccnn(pts, feats, pdf, smp, neigh, ends, radii, kp, sigma, w)) < FWD_TOL
    _check(ops.pccnn_grads(*args, t(g)),
           oracle.pccnn_grads(pts, feats, pdf, smp, neigh, ends, radii, kp, sigma, w, g),
           ("dW", "dFeat", "dKernelPts", "dPdf", "dPts", "dSamples"))
    var = ops.pccnn_weight_variance(*args[:-1])
    exp = oracle.pccnn_weight_var(pts, feats, pdf, smp, neigh, ends, radii, kp, sigma)
    assert abs(float(var) - float(exp)) < 1e-5 * abs(float(exp))


@pytest.mark.parametrize("k,c_in,c_out,distinct", [(16, 32, 24, True), (8, 5, 7, False), (24, 64, 16, True)])
def test_pointconv_basis_and_conv(ops, oracle, k, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 100 + k, distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    axis = rng.normal(0, np.sqrt(1 / 3), (3, k)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, k)).astype(np.float32)
    d = nb["dev"]
    bargs = (d["pts"], d["radii"], d["samples"], d["neigh"], t(axis), t(bias))
    basis = ops.point_conv_basis(*bargs)
    exp_basis, _ = oracle.pointconv_basis(pts, radii, smp, neigh, axis, bias)
    assert tuple(basis.shape) == exp_basis.shape and relerr(basis.cpu().numpy(), exp_basis) < FWD_TOL
    gb = rng.normal(size=exp_basis.shape).astype(np.float32)
    _check(ops.point_conv_basis_grads(*bargs, t(gb)),
           oracle.pointconv_basis_grads(pts, radii, smp, neigh, axis, bias, gb),
           ("dPts", "dSamples", "dAxis", "dBias"))
    # the convolution on caller-provided basis values (here: relu of the basis times a per-pair factor)
    act = (np.maximum(exp_basis, 0) * rng.uniform(0.2, 1.0, (neigh.shape[0], 1))).astype(np.float32)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    cargs = (t(act), t(feats), d["neigh"], d["ends"], t(w))
    out = ops.point_conv(*cargs)
    assert relerr(out.cpu().numpy(), oracle.pointconv(act, feats, neigh, ends, w)) < FWD_TOL
    _check(ops.point_conv_grads(*cargs, t(g)), oracle.pointconv_grads(act, feats, neigh, ends, w, g),
           ("dW", "dFeat", "dBasis"))
    var = ops.point_conv_weight_var(*cargs[:-1])
    exp = oracle.pointconv_weight_var(act, feats, neigh, ends)
    assert abs(float(var) - float(exp)) < 1e-5 * abs(float(exp))


@pytest.mark.parametrize("bins,c_in,c_out,distinct", [((3, 4, 3), 32, 24, True), ((1, 2, 2), 5, 7, False),
                                                      ((3, 7, 3), 16, 8, True)])
def test_sphconv_forward_and_grads(ops, oracle, bins, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 120 + bins[1], distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    radial = np.linspace(0, 1, bins[0] + 1)[1:].astype(np.float32)
    azimuth = np.linspace(-np.pi / 2, np.pi / 2, bins[1] + 1)[1:].astype(np.float32)
    polar = np.linspace(0, np.pi, bins[2] + 1)[1:].astype(np.float32)
    k = bins[0] * bins[1] * bins[2] + 1
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    d = nb["dev"]
    args = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(radial), t(azimuth), t(polar), t(w))
    out = ops.sph_conv(*args)
    exp = oracle.sphconv(pts, feats, smp, neigh, ends, radii, radial, azimuth, polar, w)
    assert relerr(out.cpu().numpy(), exp) < FWD_TOL
    _check(ops.sph_conv_grads(*args, t(g)),
           oracle.sphconv_grads(pts, feats, smp, neigh, ends, radii, radial, azimuth, polar, w, g), ("dW", "dFeat"))
    var = ops.sph_conv_weight_var(*args[:-1])
    exp = oracle.sphconv_weight_var(pts, feats, smp, neigh, ends, radii, radial, azimuth, polar)
    assert abs(float(var) - float(exp)) < 1e-5 * abs(float(exp))


def test_generic_entry_point_equals_dedicated_ones(ops):
    # pccnn_conv_forward with a KP / MLP descriptor runs the same kernels as pccnn_kpconv_forward / pccnn_mcconv_forward.
    pts, smp, nb, rng = _case(ops, 7, True, num_pts=600)
    d = nb["dev"]
    k, c_in, c_out = 16, 8, 12
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    feats, w = t(rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)), t(rng.normal(size=(k * c_in, c_out)).astype(np.float32))
    tkp = t(kp)
    ref = ops.kp_conv(d["pts"], feats, d["samples"], d["neigh"], d["ends"], d["radii"], tkp, sigma, w)
    desc = ops._basis(ops.BASIS_KP, k, tkp, sigma=sigma)
    out = ops._generic_forward("generic", desc, k, d["pts"], feats, d["samples"], d["neigh"], d["ends"], d["radii"], w,
                               False, False)
    assert torch.equal(ref, out)
    pdf = t(rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32))
    axis, bias = t(rng.normal(size=(3, k)).astype(np.float32)), t(rng.normal(size=(1, k)).astype(np.float32))
    ref = ops.mc_conv(d["pts"], pdf, feats, d["samples"], d["neigh"], d["ends"], d["radii"], axis, bias, w.reshape(1, -1, c_out))
    desc = ops._basis(ops.BASIS_MLP, k, axis, bias, pdf=pdf)
    out = ops._generic_forward("generic", desc, k, d["pts"], feats, d["samples"], d["neigh"], d["ends"], d["radii"], w,
                               False, False)
    assert torch.equal(ref, out)


def test_families_empty_and_error_paths(ops):
    pts, smp, nb, rng = _case(ops, 9, False, num_pts=200)
    d = nb["dev"]
    feats = torch.zeros((pts.shape[0], 4), device=DEV)
    kp = torch.zeros((8, 3), device=DEV)
    pdf = torch.ones(pts.shape[0], device=DEV)
    with pytest.raises(RuntimeError, match="pdf"):
        ops.kp_conv_n(d["pts"], pdf[:-1].contiguous(), feats, d["samples"], d["neigh"], d["ends"], d["radii"], kp, 0.3,
                      torch.zeros((32, 2), device=DEV))
    with pytest.raises(RuntimeError, match="sigma"):
        ops.pccnn(d["pts"], feats, pdf, d["samples"], d["neigh"], d["ends"], d["radii"], kp, 0.0,
                  torch.zeros((32, 2), device=DEV))
    with pytest.raises(RuntimeError, match="outside"):
        ops.sph_conv(d["pts"], feats, d["samples"], d["neigh"], d["ends"], d["radii"], torch.ones(4, device=DEV),
                     torch.ones(4, device=DEV), torch.ones(4, device=DEV), torch.zeros((65 * 4, 2), device=DEV))
    with pytest.raises(RuntimeError, match="basis must be"):
        ops.point_conv(torch.zeros((3, 8), device=DEV), feats, d["neigh"], d["ends"], torch.zeros((32, 2), device=DEV))
    # no pairs at all: outputs and gradients are zeros of the right shapes
    none = torch.zeros((0, 2), dtype=torch.int32, device=DEV)
    ends0 = torch.zeros(pts.shape[0], dtype=torch.int32, device=DEV)
    w = torch.ones((32, 2), device=DEV)
    out = ops.point_conv(torch.zeros((0, 8), device=DEV), feats, none, ends0, w)
    assert tuple(out.shape) == (pts.shape[0], 2) and float(out.abs().max()) == 0.0
    out = ops.sph_conv(d["pts"], feats, d["samples"], none, ends0, d["radii"], torch.ones(1, device=DEV),
                       torch.ones(1, device=DEV), torch.ones(1, device=DEV), torch.ones((8, 2), device=DEV))
    assert float(out.abs().max()) == 0.0
    grads = ops.point_conv_basis_grads(d["pts"], d["radii"], d["samples"], none, torch.ones((3, 8), device=DEV),
                                       torch.zeros((1, 8), device=DEV), torch.zeros((0, 8), device=DEV))
    assert all(float(g.abs().max()) == 0.0 for g in grads)


# --------------------------------------------------------------------------- layer modules

def _layer_case(seed, c_in):
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(seed, 2, 1200)
    rng = np.random.default_rng(seed)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pc.compute_pdf(np.full(3, 0.02, np.float32))
    return lib, pts, feats, pc, rng


def _host(x):
    return x.detach().cpu().numpy()


@pytest.mark.parametrize("kind", ["KPConvN", "PCCNN"])
def test_density_kernel_point_layers(oracle, kind):
    lib, pts, feats, pc, rng = _layer_case(31, 16)
    torch.manual_seed(3)
    layer = getattr(lib.pc.layers, kind)(3, 16, 24, 16).to(DEV)
    tf = t(feats).requires_grad_(True)
    out, nbh = layer(pc, pc, tf, 0.1)
    g = rng.normal(size=tuple(out.shape)).astype(np.float32)
    out.backward(t(g))
    neigh, ends = _host(nbh.neighbors_), _host(nbh.start_ids_)
    radii = np.full(3, 0.1, np.float32)
    pdf = _host(pc.pts_unnorm_pdf_ * torch.prod(t(radii)))
    kp, sigma, w = _host(layer.kernel_pts_), float(layer.sigma_.item()), _host(layer.conv_weights_)
    if kind == "KPConvN":
        exp = oracle.kpconvn(pts, pdf, feats, pts, neigh, ends, radii, kp, sigma, w)
        exp_g = oracle.kpconvn_grads(pts, pdf, feats, pts, neigh, ends, radii, kp, sigma, w, g)
    else:
        exp = oracle.pccnn(pts, feats, pdf, pts, neigh, ends, radii, kp, sigma, w)
        exp_g = oracle.pccnn_grads(pts, feats, pdf, pts, neigh, ends, radii, kp, sigma, w, g)
    assert relerr(_host(out), exp) < FWD_TOL
    assert relerr(_host(layer.conv_weights_.grad), exp_g[0]) < GRAD_TOL
    assert relerr(_host(tf.grad), exp_g[1]) < GRAD_TOL
    # variance-aware initialisation: the statistic of the warm-up pass is the op's
    factory = getattr(lib.pc.layers, kind + "Factory")(16, True)
    warm = factory.create_conv_layer(3, 16, 24).to(DEV)
    factory.set_init_warmup_state_convs(True)
    warm(pc, pc, t(feats), 0.1, nbh)
    var = (oracle.kpconvn_weight_var(pts, pdf, feats, pts, neigh, ends, radii, _host(warm.kernel_pts_),
                                     float(warm.sigma_.item())) if kind == "KPConvN" else
           oracle.pccnn_weight_var(pts, feats, pdf, pts, neigh, ends, radii, _host(warm.kernel_pts_),
                                   float(warm.sigma_.item())))
    assert abs(warm.accum_weight_var_ - 1.0 / float(var)) < 1e-4 * abs(1.0 / float(var))


def test_sphconv_layer(oracle):
    lib, pts, feats, pc, rng = _layer_case(32, 8)
    torch.manual_seed(4)
    layer = lib.pc.layers.SPHConvFactory(2, 5, 3).create_conv_layer(3, 8, 12).to(DEV)
    assert layer.num_basis_ == 31 and tuple(layer.conv_weights_.shape) == (31 * 8, 12)
    tf = t(feats).requires_grad_(True)
    out, nbh = layer(pc, pc, tf, 0.1)
    g = rng.normal(size=tuple(out.shape)).astype(np.float32)
    out.backward(t(g))
    neigh, ends = _host(nbh.neighbors_), _host(nbh.start_ids_)
    radii = np.full(3, 0.1, np.float32)
    bins = [_host(b) for b in (layer.radial_bins_, layer.azimuz_bins_, layer.polar_bins_)]
    w = _host(layer.conv_weights_)
    assert relerr(_host(out), oracle.sphconv(pts, feats, pts, neigh, ends, radii, *bins, w)) < FWD_TOL
    exp_g = oracle.sphconv_grads(pts, feats, pts, neigh, ends, radii, *bins, w, g)
    assert relerr(_host(layer.conv_weights_.grad), exp_g[0]) < GRAD_TOL
    assert relerr(_host(tf.grad), exp_g[1]) < GRAD_TOL


@pytest.mark.parametrize("norm", ["none", "bn", "gn"])
def test_pointconv_layer(oracle, norm):
    lib, pts, feats, pc, rng = _layer_case(33, 8)
    torch.manual_seed(5)
    layer = lib.pc.layers.PointConvFactory(16, False, 1.0, norm == "bn", norm == "gn", 4) \
        .create_conv_layer(3, 8, 12).to(DEV)
    layer.proj_bias_.data.normal_(0, 0.1)
    tf = t(feats).requires_grad_(True)
    out, nbh = layer(pc, pc, tf, 0.1)
    g = rng.normal(size=tuple(out.shape)).astype(np.float32)
    out.backward(t(g))
    # (as in the reference, the group norm of the basis never feeds the output, so its parameters get no gradient)
    assert all(p.grad is not None and torch.isfinite(p.grad).all()
               for n, p in layer.named_parameters() if not n.startswith("basis_gn_"))
    if norm != "none":
        return
    # without normalisation layers the module is: basis op -> relu -> * density network -> conv op
    neigh, ends = _host(nbh.neighbors_), _host(nbh.start_ids_)
    scale = _host(layer.__density_scale__(pc, nbh))
    assert scale.shape == (neigh.shape[0], 1) and 0.0 < scale.min() and scale.max() < 1.0
    basis, _ = oracle.pointconv_basis(pts, np.ones(3, np.float32), pts, neigh, _host(layer.proj_axis_),
                                      _host(layer.proj_bias_))
    act = (np.maximum(basis, 0) * scale).astype(np.float32)
    w = _host(layer.conv_weights_)
    assert relerr(_host(out), oracle.pointconv(act, feats, neigh, ends, w)) < 2e-5
    exp_g = oracle.pointconv_grads(act, feats, neigh, ends, w, g)
    assert relerr(_host(layer.conv_weights_.grad), exp_g[0]) < GRAD_TOL
    assert relerr(_host(tf.grad), exp_g[1]) < GRAD_TOL
    # the basis gradient flows on through relu and the basis op into the projection parameters
    dbasis = exp_g[2] * scale * (basis > 0)
    exp_b = oracle.pointconv_basis_grads(pts, np.ones(3, np.float32), pts, neigh, _host(layer.proj_axis_),
                                         _host(layer.proj_bias_), dbasis.astype(np.float32))
    assert relerr(_host(layer.proj_axis_.grad), exp_b[2]) < GRAD_TOL
    assert relerr(_host(layer.proj_bias_.grad), exp_b[3]) < GRAD_TOL


def test_group_normalization_and_bias():
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(3, 3, 200)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    feats = torch.randn((600, 8), device=DEV) * 3 + 1
    gn = lib.pc.layers.GroupNormalization(8, 4).to(DEV)
    out = gn(feats, pc).detach()
    # per cloud and group column the normalised values have zero mean and unit variance
    view = out.reshape(-1, 4)
    vid = pc.batch_ids_.reshape(-1, 1).repeat(1, 2).reshape(-1).to(torch.int64)
    for b in range(3):
        sel = view[vid == b]
        assert float(sel.mean(dim=0).abs().max()) < 1e-5 and float((sel.var(dim=0, unbiased=False) - 1).abs().max()) < 1e-4
    bias = lib.pc.layers.Bias(8).to(DEV)
    bias.bias_.data.fill_(0.5)
    assert torch.equal(bias(feats), feats + 0.5)
