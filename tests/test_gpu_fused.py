"""The optional forward convolution that keeps the projection on chip (one kernel from the gather to the output)
against the oracle and against the two-kernel path, through the op module: with set_fused_forward(True) a forward
call that does not return its projection takes it when the shape allows."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, relerr, t

pytestmark = pytest.mark.gpu

FWD_TOL = 1e-5


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _case(ops, seed, batch, num_pts, radius, distinct, far_samples=0):
    pts, ids = synthetic.primitives(seed, batch, num_pts)
    rng = np.random.default_rng(seed)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    if far_samples:
        # samples in an empty corner of the first cloud's box: no neighbors, rows of zeros
        lo = pts[ids == 0].min(axis=0)
        extra = (lo + 1e-4 * rng.random((far_samples, 3))).astype(np.float32)
        smp = np.concatenate([extra, smp]).astype(np.float32)
        sids = np.concatenate([np.zeros(far_samples, np.int32), sids])
    nb = gpu_neighborhood(ops, pts, ids, smp, sids, radius, batch)
    return pts, smp, nb, rng


def _both_paths(ops, call):
    """The same forward call with the fused path on and off; returns (fused, two-kernel) outputs and checks, through
    the library's own launch counters, that the first really ran fused and the second did not."""
    from pccnn_lib_amd import _lib
    outs = []
    for fused in (True, False):
        before = ops.set_fused_forward(fused)
        try:
            _lib.timing(enable=True, reset=True)
            outs.append(call())
            torch.cuda.synchronize()
            timers = _lib.timing(enable=False)
        finally:
            ops.set_fused_forward(before)
        assert ("fused_fwd" in timers) == fused and ("proj_fwd" in timers) == (not fused), timers
    return outs


@pytest.mark.parametrize("c_in,hidden,c_out,distinct,radius", [(64, 16, 128, False, 0.12), (128, 8, 64, True, 0.12),
                                                               (48, 6, 256, True, 0.15), (64, 16, 128, True, 0.5)])
def test_fused_mcconv_forward(ops, oracle, c_in, hidden, c_out, distinct, radius):
    # (the radius of 0.5 gives samples several hundred neighbors: more than one staging batch per sample)
    pts, smp, nb, rng = _case(ops, 300 + c_in + hidden, 2, 1100, radius, distinct, far_samples=5 if distinct else 0)
    d = nb["dev"]
    n = pts.shape[0]
    pdf = rng.uniform(0.5, 2.0, n).astype(np.float32)
    feats = rng.normal(size=(n, c_in)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, hidden)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * hidden)), (1, hidden * c_in, c_out)).astype(np.float32)
    args = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(w))
    fused, plain = _both_paths(ops, lambda: ops.mc_conv(*args))
    exp = oracle.mcconv(pts, pdf, feats, smp, nb["neighbors"], nb["ends"], nb["radii"], axis, bias, w)
    assert relerr(fused.cpu().numpy(), exp) < FWD_TOL
    assert relerr(fused.cpu().numpy(), plain.cpu().numpy()) < FWD_TOL
    if distinct and radius < 0.2:
        assert nb["ends"][4] == 0 and float(fused[:5].abs().max()) == 0.0          # the samples without neighbors
    # a call that returns its projection keeps the two-kernel path, and gives the same output
    out, proj = ops.mc_conv(*args, return_proj=True)
    assert torch.equal(out, plain) and tuple(proj.shape) == (smp.shape[0], c_in, hidden)


@pytest.mark.parametrize("k,c_in,c_out", [(15, 128, 256), (16, 64, 64), (9, 40, 128)])
def test_fused_kpconv_forward(ops, oracle, k, c_in, c_out):
    pts, smp, nb, rng = _case(ops, 400 + k, 2, 1333, 0.12, k != 16)
    d = nb["dev"]
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    args = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    fused, plain = _both_paths(ops, lambda: ops.kp_conv(*args))
    exp = oracle.kpconv(pts, feats, smp, nb["neighbors"], nb["ends"], nb["radii"], kp, sigma, w)
    assert relerr(fused.cpu().numpy(), exp) < FWD_TOL
    assert relerr(fused.cpu().numpy(), plain.cpu().numpy()) < FWD_TOL


def test_shapes_outside_the_fused_kernel_take_the_two_kernel_path(ops):
    # more than 16 basis functions, few input features, other output widths, several MLPs: two kernels, as before
    from pccnn_lib_amd import _lib
    pts, smp, nb, rng = _case(ops, 450, 1, 900, 0.15, False)
    d = nb["dev"]
    before = ops.set_fused_forward(True)
    assert before is False                              # off unless asked for
    try:
        for k, c_in, c_out in ((33, 64, 128), (16, 32, 128), (16, 64, 96)):
            kp, sigma = synthetic.kernel_points_sphere(1, k)
            feats = t(rng.normal(size=(pts.shape[0], c_in)).astype(np.float32))
            w = t(rng.normal(0, 0.05, (k * c_in, c_out)).astype(np.float32))
            _lib.timing(enable=True, reset=True)
            ops.kp_conv(d["pts"], feats, d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, w)
            torch.cuda.synchronize()
            timers = _lib.timing(enable=False)
            assert "fused_fwd" not in timers and "proj_fwd" in timers, (k, c_in, c_out)
        # two MLPs (MCConv with the feature axis split over two weight blocks)
        n, c_in, hidden, c_out = pts.shape[0], 64, 8, 128
        feats = t(rng.normal(size=(n, c_in)).astype(np.float32))
        pdf = t(rng.uniform(0.5, 2.0, n).astype(np.float32))
        axis = t(rng.normal(0, 0.6, (3, 2 * hidden)).astype(np.float32))
        bias = t(rng.normal(0, 0.1, (1, 2 * hidden)).astype(np.float32))
        w = t(rng.normal(0, 0.05, (2, hidden * c_in, c_out // 2)).astype(np.float32))
        _lib.timing(enable=True, reset=True)
        out = ops.mc_conv(d["pts"], pdf, feats, d["samples"], d["neigh"], d["ends"], d["radii"], axis, bias, w)
        torch.cuda.synchronize()
        timers = _lib.timing(enable=False)
        assert "fused_fwd" not in timers and "proj_fwd" in timers and tuple(out.shape) == (n, c_out)
    finally:
        ops.set_fused_forward(before)


def test_fused_forward_of_the_other_families(ops, oracle):
    pts, smp, nb, rng = _case(ops, 500, 2, 1200, 0.12, True)
    d = nb["dev"]
    n = pts.shape[0]
    c_in, c_out, k = 64, 128, 16
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    pdf = rng.uniform(0.5, 2.0, n).astype(np.float32)
    feats = rng.normal(size=(n, c_in)).astype(np.float32)
    w = rng.normal(0, 0.05, (k * c_in, c_out)).astype(np.float32)
    geo = (d["samples"], d["neigh"], d["ends"], d["radii"])
    host = (smp, nb["neighbors"], nb["ends"], nb["radii"])
    fused, plain = _both_paths(ops, lambda: ops.kp_conv_n(d["pts"], t(pdf), t(feats), *geo, t(kp), sigma, t(w)))
    assert relerr(fused.cpu().numpy(), oracle.kpconvn(pts, pdf, feats, *host, kp, sigma, w)) < FWD_TOL
    fused, plain = _both_paths(ops, lambda: ops.pccnn(d["pts"], t(feats), t(pdf), *geo, t(kp), sigma, t(w)))
    assert relerr(fused.cpu().numpy(), oracle.pccnn(pts, feats, pdf, *host, kp, sigma, w)) < FWD_TOL
    # a caller-given basis (PointConv)
    axis = rng.normal(0, 0.6, (3, k)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, k)).astype(np.float32)
    basis = ops.point_conv_basis(d["pts"], d["radii"], d["samples"], d["neigh"], t(axis), t(bias))
    fused, plain = _both_paths(ops, lambda: ops.point_conv(basis, t(feats), d["neigh"], d["ends"], t(w)))
    exp = oracle.pointconv(basis.cpu().numpy(), feats, nb["neighbors"], nb["ends"], w)
    assert relerr(fused.cpu().numpy(), exp) < FWD_TOL
    assert relerr(fused.cpu().numpy(), plain.cpu().numpy()) < FWD_TOL


def test_fused_forward_with_bf16_operands(ops, oracle):
    pts, smp, nb, rng = _case(ops, 600, 2, 1500, 0.12, False)
    d = nb["dev"]
    n = pts.shape[0]
    c_in, hidden, c_out = 64, 16, 128
    pdf = rng.uniform(0.5, 2.0, n).astype(np.float32)
    feats = rng.normal(size=(n, c_in)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, hidden)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * hidden)), (1, hidden * c_in, c_out)).astype(np.float32)
    args = (d["pts"], t(pdf), t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(axis), t(bias), t(w))
    fused, plain = _both_paths(ops, lambda: ops.mc_conv(*args, contraction="bf16"))
    exp = oracle.mcconv(pts, pdf, feats, smp, nb["neighbors"], nb["ends"], nb["radii"], axis, bias, w,
                        contraction="bf16")
    # same rounded operands, fp32 accumulation in another order; an entry of the projection on a bf16 rounding
    # boundary may round the other way in one of the three
    assert relerr(fused.cpu().numpy(), exp) < 1e-3
    assert relerr(fused.cpu().numpy(), plain.cpu().numpy()) < 1e-3
    assert relerr(fused.cpu().numpy(), oracle.mcconv(pts, pdf, feats, smp, nb["neighbors"], nb["ends"], nb["radii"],
                                                     axis, bias, w)) < 3e-2


def test_layers_take_the_fused_path_without_gradients(ops, oracle):
    # a layer called under torch.no_grad() keeps no projection: with the fused path switched on, one kernel per convolution
    import pccnn_lib_amd as lib
    from pccnn_lib_amd import _lib
    pts, ids = synthetic.primitives(77, 2, 1500)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    pc.compute_pdf(np.full(3, 0.02, np.float32))
    torch.manual_seed(3)
    layer = lib.pc.layers.MCConv(3, 64, 128, 16).to(DEV)
    feats = torch.randn(pts.shape[0], 64, device=DEV)
    out_grad, nbh = layer(pc, pc, feats.clone().requires_grad_(True), 0.1)
    before = ops.set_fused_forward(True)
    try:
        _lib.timing(enable=True, reset=True)
        with torch.no_grad():
            out = layer(pc, pc, feats, 0.1, nbh)
        torch.cuda.synchronize()
        timers = _lib.timing(enable=False)
    finally:
        ops.set_fused_forward(before)
    assert "fused_fwd" in timers and "proj_fwd" not in timers and "gemm" not in timers
    assert relerr(out.cpu().numpy(), out_grad.detach().cpu().numpy()) < FWD_TOL
