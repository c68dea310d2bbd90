"""The backward pass without float atomics (GRAD_DETERMINISTIC): feature gradients stored per pair and summed per
point in a fixed order, point-side gradients by the same index, basis-parameter partial sums per sample.  Every
gradient must equal the oracle's (the same bar as the default pass) and be bit-identical from run to run."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, mixed_close, relerr, t

pytestmark = pytest.mark.gpu

GRAD_TOL = 1e-4


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _case(ops, seed, num_pts, radius, distinct):
    pts, ids = synthetic.primitives(seed, 2, num_pts)
    rng = np.random.default_rng(seed)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    return pts, smp, gpu_neighborhood(ops, pts, ids, smp, sids, radius, 2), rng


def _identical_runs(call, runs=3):
    first = call()
    for _ in range(runs - 1):
        again = call()
        for a, b in zip(first, again):
            assert (a is None) == (b is None)
            if a is not None:
                assert torch.equal(a, b)
    return first


@pytest.mark.parametrize("c_in,hidden,c_out,distinct,with_mirror", [(64, 16, 128, False, True), (64, 16, 128, False, False),
                                                                    (8, 8, 32, True, False), (24, 4, 16, True, False)])
def test_mcconv_gradients_without_atomics(ops, oracle, c_in, hidden, c_out, distinct, with_mirror):
    # (8 and 24 input features take the pair-parallel kernels for few features)
    pts, smp, nb, rng = _case(ops, 700 + c_in + hidden, 1300, 0.12, distinct)
    d = nb["dev"]
    n = pts.shape[0]
    pdf = rng.uniform(0.5, 2.0, n).astype(np.float32)
    feats = rng.normal(size=(n, c_in)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, hidden)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * hidden)), (1, hidden * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    args = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(w), t(g))
    mirror = ops.mirror_pairs(d["neigh"], d["ends"]) if with_mirror else None
    assert (mirror is not None) == with_mirror
    grads = _identical_runs(lambda: ops.mc_conv_grads(*args, grad_mask=ops.GRAD_ALL | ops.GRAD_DETERMINISTIC,
                                                      mirror=mirror))
    exp = oracle.mcconv_grads(pts, pdf, feats, smp, nb["neighbors"], nb["ends"], nb["radii"], axis, bias, w, g)
    for got, e, name in zip(grads, exp, ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < GRAD_TOL, name
        assert mixed_close(got.cpu().numpy(), e), name
    # a subset of the groups, and the same with bf16 contraction operands
    part = _identical_runs(lambda: ops.mc_conv_grads(*args, grad_mask=ops.GRAD_FEATS | ops.GRAD_DETERMINISTIC,
                                                     mirror=mirror))
    assert part[0] is None and torch.equal(part[1], grads[1])
    b16 = _identical_runs(lambda: ops.mc_conv_grads(*args, grad_mask=ops.GRAD_ALL | ops.GRAD_DETERMINISTIC, mirror=mirror,
                                                    contraction="bf16"))
    exp16 = oracle.mcconv_grads(pts, pdf, feats, smp, nb["neighbors"], nb["ends"], nb["radii"], axis, bias, w, g,
                                contraction="bf16")
    for got, e, name in zip(b16, exp16, ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")):
        assert relerr(got.cpu().numpy(), e) < 1e-3, name


@pytest.mark.parametrize("k,c_in,c_out,distinct", [(15, 128, 64, False), (16, 40, 24, True)])
def test_kpconv_gradients_without_atomics(ops, oracle, k, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 800 + k, 1200, 0.12, distinct)
    d = nb["dev"]
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    args = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w), t(g))
    grads = _identical_runs(lambda: ops.kp_conv_grads(*args, grad_mask=ops.GRAD_ALL | ops.GRAD_DETERMINISTIC))
    exp = oracle.kpconv_grads(pts, feats, smp, nb["neighbors"], nb["ends"], nb["radii"], kp, sigma, w, g)
    for got, e, name in zip(grads, exp, ("dW", "dFeat", "dKernelPts", "dPts", "dSamples")):
        assert relerr(got.cpu().numpy(), e) < GRAD_TOL, name
    # the default pass gives the same numbers up to the order of its atomic additions
    plain = ops.kp_conv_grads(*args)
    for a, b in zip(grads, plain):
        assert relerr(a.cpu().numpy(), b.cpu().numpy()) < 1e-5


def test_pointconv_gradients_without_atomics(ops, oracle):
    pts, smp, nb, rng = _case(ops, 900, 1100, 0.12, True)
    d = nb["dev"]
    k, c_in, c_out = 16, 48, 32
    basis = t(rng.normal(size=(nb["neighbors"].shape[0], k)).astype(np.float32))
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, 0.05, (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    grads = _identical_runs(lambda: ops.point_conv_grads(basis, t(feats), d["neigh"], d["ends"], t(w), t(g),
                                                         grad_mask=ops.GRAD_ALL | ops.GRAD_DETERMINISTIC))
    exp = oracle.pointconv_grads(basis.cpu().numpy(), feats, nb["neighbors"], nb["ends"], w, g)
    for got, e, name in zip(grads, exp, ("dW", "dFeat", "dBasis")):
        assert relerr(got.cpu().numpy(), e) < GRAD_TOL, name


@pytest.mark.parametrize("c_in", [40, 12])
def test_the_other_families_without_atomics(ops, oracle, c_in):
    # KPConvN, PCCNN (both divide by the density) and SPHConv (bins, no geometry gradients): same bar, same bits
    # from run to run; 12 features take the pair-parallel kernels
    pts, smp, nb, rng = _case(ops, 950 + c_in, 1000, 0.12, True)
    d = nb["dev"]
    n, k, c_out = pts.shape[0], 16, 24
    kp, sigma = synthetic.kernel_points_sphere(2, k)
    pdf = rng.uniform(0.5, 2.0, n).astype(np.float32)
    feats = rng.normal(size=(n, c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    geo = (d["samples"], d["neigh"], d["ends"], d["radii"])
    host = (smp, nb["neighbors"], nb["ends"], nb["radii"])
    mask = ops.GRAD_ALL | ops.GRAD_DETERMINISTIC
    got = _identical_runs(lambda: ops.kp_conv_n_grads(d["pts"], t(pdf), t(feats), *geo, t(kp), sigma, t(w), t(g),
                                                      grad_mask=mask))
    exp = oracle.kpconvn_grads(pts, pdf, feats, *host, kp, sigma, w, g)
    for a, e, name in zip(got, exp, ("dW", "dFeat", "dKernelPts", "dPts", "dSamples")):
        assert relerr(a.cpu().numpy(), e) < GRAD_TOL, name
    got = _identical_runs(lambda: ops.pccnn_grads(d["pts"], t(feats), t(pdf), *geo, t(kp), sigma, t(w), t(g),
                                                  grad_mask=mask))
    exp = oracle.pccnn_grads(pts, feats, pdf, *host, kp, sigma, w, g)
    for a, e, name in zip(got, exp, ("dW", "dFeat", "dKernelPts", "dPdf", "dPts", "dSamples")):
        assert relerr(a.cpu().numpy(), e) < GRAD_TOL, name
    radial = np.linspace(0, 1, 4)[1:].astype(np.float32)
    azimuth = np.linspace(-np.pi / 2, np.pi / 2, 5)[1:].astype(np.float32)
    polar = np.linspace(0, np.pi, 4)[1:].astype(np.float32)
    ks = 3 * 4 * 3 + 1
    ws = rng.normal(0, np.sqrt(1.0 / (ks * c_in)), (ks * c_in, c_out)).astype(np.float32)
    got = _identical_runs(lambda: ops.sph_conv_grads(d["pts"], t(feats), *geo, t(radial), t(azimuth), t(polar), t(ws),
                                                     t(g), grad_mask=ops.GRAD_WEIGHTS | ops.GRAD_FEATS
                                                     | ops.GRAD_DETERMINISTIC))
    exp = oracle.sphconv_grads(pts, feats, *host, radial, azimuth, polar, ws, g)
    for a, e, name in zip(got, exp, ("dW", "dFeat")):
        assert relerr(a.cpu().numpy(), e) < GRAD_TOL, name


def test_layers_give_identical_gradients_from_run_to_run_when_asked(ops, oracle):
    # set_deterministic(True): the autograd wrappers ask for the pass without atomics; two passes over a level of a
    # hierarchy (pooled samples: no mirror index) and over a symmetric neighborhood give the same bits
    import pccnn_lib_amd as lib
    pts, ids = synthetic.primitives(91, 2, 2500)
    torch.manual_seed(9)
    layer_a = lib.pc.layers.MCConv(3, 16, 64, 8).to(DEV)
    layer_b = lib.pc.layers.KPConv(3, 64, 32, 15).to(DEV)
    feats0 = torch.randn(pts.shape[0], 16, device=DEV)

    def run():
        pc = lib.pc.Pointcloud(t(pts).clone().requires_grad_(True), t(ids))
        with torch.no_grad():           # (the density's own gradient op adds with atomics, like the reference's)
            pc.compute_pdf(0.02)
        pool = lib.pc.PointPooling(pc, 0.05)
        out_pc = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
        feats = feats0.clone().requires_grad_(True)
        mid, _ = layer_a(pc, out_pc, feats, 0.1)
        out, _ = layer_b(out_pc, out_pc, torch.nn.functional.leaky_relu(mid, 0.2), 0.15)
        params = [layer_a.conv_weights_, layer_a.proj_axis_, layer_a.proj_bias_, layer_b.conv_weights_]
        return torch.autograd.grad((out * out).sum(), [feats, pc.pts_] + params)

    before = ops.set_deterministic(True)
    try:
        assert before is False and ops.deterministic_flag() == ops.GRAD_DETERMINISTIC
        first, second = run(), run()
    finally:
        ops.set_deterministic(before)
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    plain = run()
    for a, b in zip(first, plain):
        assert relerr(a.cpu().numpy(), b.cpu().numpy()) < 1e-5


def test_the_pass_without_atomics_is_three_dimensional(ops):
    rng = np.random.default_rng(4)
    pts = rng.random((800, 4), dtype=np.float32)
    ids = np.zeros(800, np.int32)
    nb = gpu_neighborhood(ops, pts, ids, pts, ids, 0.3, 1)["dev"]
    kp = t(rng.normal(0, 0.3, (8, 4)).astype(np.float32))
    feats, w, g = torch.randn(800, 8, device=DEV), torch.randn(64, 8, device=DEV), torch.randn(800, 8, device=DEV)
    with pytest.raises(RuntimeError, match="three-dimensional"):
        ops.kp_conv_grads(nb["pts"], feats, nb["samples"], nb["neigh"], nb["ends"], nb["radii"], kp, 0.3, w, g,
                          grad_mask=ops.GRAD_ALL | ops.GRAD_DETERMINISTIC)
