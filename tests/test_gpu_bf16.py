"""The bf16 contraction mode (bf16 operands, fp32 accumulation; config 5 of the baseline) against the CPU oracle.

The reference has no such mode, so the bar is the oracle with the same operand rounding (`contraction="bf16"`:
projection, weights and incoming gradients rounded to the nearest bf16, products summed in float64):

* the projection the HIP path hands back must equal the oracle's rounded projection except for the rare entries
  whose fp32 sum sits on a bf16 rounding boundary (the two sides add the pairs in different orders), and those
  may differ by one bf16 step only;
* output and weight gradients must equal the products of that very projection with the rounded weights / incoming
  gradients to the fp32 tolerances (1e-5 / 1e-4): this pins the matrix kernel and the rounding exactly;
* every other gradient does not involve the projection and must match the oracle to 1e-4;
* end to end, results stay within BF16_TOL of the bf16 oracle and within LOOSE_TOL (what 8 bits of operand
  mantissa allow) of the plain fp32 oracle."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic
from tests.gpu_helpers import DEV, gpu_neighborhood, relerr, t

pytestmark = pytest.mark.gpu

FWD_TOL = 1e-5
GRAD_TOL = 1e-4
BF16_TOL = 3e-3      # relative to the largest magnitude of the tensor; a flipped projection entry costs up to ~2e-3
LOOSE_TOL = 3e-2


def _check_projection(oracle, proj_gpu, proj_oracle):
    """bf16 projection from the HIP path vs the oracle's fp32 projection rounded to bf16."""
    got = proj_gpu.to(torch.float32).cpu().numpy()
    exp = oracle.bf16_round(proj_oracle)
    diff = got != exp
    assert diff.mean() < 2e-3, "too many projection entries round differently: %g" % diff.mean()
    # one bf16 step is at most 2^-7 of the value; entries that are small against the terms they sum carry the
    # fp32 summation difference of the two sides on top
    step = np.abs(exp) * 2.0 ** -7 + 1e-5 * np.abs(exp).max()
    assert np.all(np.abs(got - exp)[diff] <= step[diff])
    return got


def _products(proj, w, g):
    """out and dW of the contraction from a given projection [M, Cin, K], weights [mlps, inner, co] and
    incoming gradients [M, Cout], in float64 (operands as they are)."""
    m, mlps = proj.shape[0], w.shape[0]
    pr = proj.reshape(m, mlps, -1).transpose(1, 0, 2).astype(np.float64)
    out = np.matmul(pr, w.astype(np.float64)).transpose(1, 0, 2).reshape(m, -1)
    gr = g.reshape(m, mlps, -1).transpose(1, 0, 2).astype(np.float64)
    return out, np.matmul(pr.transpose(0, 2, 1), gr)


@pytest.fixture(scope="module")
def ops():
    from pccnn_lib_amd import pccnn_lib_ops
    return pccnn_lib_ops


def _stream():
    from pccnn_lib_amd import _lib
    return _lib.P(torch.cuda.current_stream().cuda_stream)


def test_rounding_matches_oracle_bit_for_bit(oracle):
    from pccnn_lib_amd import _lib
    rng = np.random.default_rng(0)
    a = (rng.normal(size=50000) * 10.0 ** rng.integers(-20, 20, 50000)).astype(np.float32)
    a[:8] = [0.0, -0.0, 1.0, 1.00390625, 1.001953125, 1.005859375, np.inf, -np.inf]    # ties and specials
    ta = t(a)
    out = torch.empty(a.shape, dtype=torch.bfloat16, device=DEV)
    _lib.call("pccnn_f32_to_bf16", _lib.P(ta.data_ptr()), _lib.P(out.data_ptr()), a.shape[0], _stream())
    torch.cuda.synchronize()
    got = out.to(torch.float32).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.bf16_round(a).view(np.uint32))


@pytest.mark.parametrize("rows,cols,inner,at,bt,split", [
    (256, 128, 64, 0, 0, 1), (256, 128, 64, 0, 1, 1), (256, 128, 64, 1, 0, 1), (256, 128, 64, 1, 1, 1),
    (300, 70, 45, 0, 0, 1), (77, 130, 19, 0, 1, 1), (129, 129, 17, 1, 1, 1), (480, 40, 1000, 1, 0, 4),
    (128, 128, 4096, 1, 0, 8), (2048, 128, 1024, 0, 0, 1), (4096, 1024, 128, 0, 1, 1), (1024, 128, 8192, 1, 0, 64),
    # edge tiles read with whole 16-byte units: the three products of a small hierarchy level
    (346, 256, 1024, 0, 0, 1), (1024, 256, 346, 1, 0, 1), (346, 1024, 256, 0, 1, 1), (512, 128, 6844, 1, 0, 64),
    (200, 72, 104, 0, 0, 1), (200, 72, 104, 1, 1, 1), (40, 8, 24, 1, 0, 1)])
def test_gemm_bf16_against_float64(oracle, rows, cols, inner, at, bt, split):
    from pccnn_lib_amd import _lib
    rng = np.random.default_rng(rows + cols + inner + at + 2 * bt)
    a = oracle.bf16_round(rng.normal(size=(inner, rows) if at else (rows, inner)).astype(np.float32))
    b = oracle.bf16_round(rng.normal(size=(cols, inner) if bt else (inner, cols)).astype(np.float32))
    ta, tb = t(a).to(torch.bfloat16), t(b).to(torch.bfloat16)          # exact: the values are bf16 already
    tc = torch.full((rows, cols), float("nan"), dtype=torch.float32, device=DEV)
    ws = torch.empty(split * rows * cols * 4 + 256, dtype=torch.uint8, device=DEV)
    _lib.call("pccnn_gemm_bf16", _lib.P(ta.data_ptr()), _lib.P(tb.data_ptr()), _lib.P(tc.data_ptr()), rows, cols, inner,
              at, bt, a.shape[1], b.shape[1], cols, 1, 0, 0, 0, split, _lib.P(ws.data_ptr()), ws.numel(), _stream())
    torch.cuda.synchronize()
    exp = (a.T if at else a).astype(np.float64) @ (b.T if bt else b).astype(np.float64)
    assert relerr(tc.cpu().numpy(), exp) < 1e-5


def test_gemm_bf16_batched_strided(oracle):
    from pccnn_lib_amd import _lib
    rng = np.random.default_rng(0)
    m, mlps, inner, co = 200, 2, 48, 24
    a = oracle.bf16_round(rng.normal(size=(m, mlps * inner)).astype(np.float32))
    b = oracle.bf16_round(rng.normal(size=(mlps, inner, co)).astype(np.float32))
    ta, tb = t(a).to(torch.bfloat16), t(b).to(torch.bfloat16)
    tc = torch.zeros((m, mlps * co), dtype=torch.float32, device=DEV)
    _lib.call("pccnn_gemm_bf16", _lib.P(ta.data_ptr()), _lib.P(tb.data_ptr()), _lib.P(tc.data_ptr()), m, co, inner, 0, 0,
              mlps * inner, co, mlps * co, mlps, inner, inner * co, co, 1, _lib.P(0), 0, _stream())
    torch.cuda.synchronize()
    exp = np.concatenate([a[:, i * inner:(i + 1) * inner].astype(np.float64) @ b[i] for i in range(mlps)], axis=1)
    assert relerr(tc.cpu().numpy(), exp) < 1e-5


def _case(ops, seed, distinct):
    pts, ids = synthetic.primitives(seed, 2, 1500)
    rng = np.random.default_rng(seed)
    if distinct:
        pick = np.sort(rng.choice(pts.shape[0], pts.shape[0] // 3, replace=False))
        smp, sids = pts[pick].copy(), ids[pick]
    else:
        smp, sids = pts, ids
    return pts, smp, gpu_neighborhood(ops, pts, ids, smp, sids, 0.12, 2), rng


@pytest.mark.parametrize("hidden,mlps,c_in,c_out,distinct", [(16, 1, 64, 128, False), (8, 2, 32, 24, True),
                                                             (16, 1, 3, 16, True)])
def test_mcconv_bf16_forward_and_grads(ops, oracle, hidden, mlps, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 140 + hidden + mlps, distinct)
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
    host = (pts, pdf, feats, smp, neigh, ends, radii, axis, bias, w)
    out, proj = ops.mc_conv(*args, return_proj=True, contraction="bf16")
    assert proj.dtype == torch.bfloat16 and tuple(proj.shape) == (smp.shape[0], c_in, k)
    basis, _ = oracle.conv_basis(oracle.MLP, pts, smp, neigh, radii, axis, bias=bias, pdf=pdf)
    proj_host = _check_projection(oracle, proj, oracle.feat_basis_proj(basis, feats, neigh, ends))
    exp_out, exp_dw = _products(proj_host, oracle.bf16_round(w), oracle.bf16_round(g))
    assert relerr(out.cpu().numpy(), exp_out) < FWD_TOL
    assert relerr(out.cpu().numpy(), oracle.mcconv(*host, contraction="bf16")) < BF16_TOL
    assert relerr(out.cpu().numpy(), oracle.mcconv(*host)) < LOOSE_TOL
    exp_g = oracle.mcconv_grads(*host, g, contraction="bf16")
    exp_f32 = oracle.mcconv_grads(*host, g)
    names = ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")
    for cached in (proj, None):                      # projection kept from the forward call, or rebuilt
        grads = ops.mc_conv_grads(*args, t(g), proj=cached, contraction="bf16")
        assert relerr(grads[0].cpu().numpy(), exp_dw.reshape(w.shape)) < GRAD_TOL
        for got, e, e32, name in zip(grads, exp_g, exp_f32, names):
            assert tuple(got.shape) == e.shape, name
            assert relerr(got.cpu().numpy(), e) < (BF16_TOL if name == "dW" else GRAD_TOL), name
            assert relerr(got.cpu().numpy(), e32) < LOOSE_TOL, name


@pytest.mark.parametrize("k,c_in,c_out,distinct", [(15, 32, 32, False), (16, 64, 48, True), (15, 5, 7, True)])
def test_kpconv_bf16_forward_and_grads(ops, oracle, k, c_in, c_out, distinct):
    pts, smp, nb, rng = _case(ops, 120 + k + c_in, distinct)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    d = nb["dev"]
    args = (d["pts"], t(feats), d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, t(w))
    host = (pts, feats, smp, neigh, ends, radii, kp, sigma, w)
    out, proj = ops.kp_conv(*args, return_proj=True, contraction="bf16")
    basis, _ = oracle.conv_basis(oracle.KP, pts, smp, neigh, radii, kp, sigma=sigma)
    proj_host = _check_projection(oracle, proj, oracle.feat_basis_proj(basis, feats, neigh, ends))
    exp_out, exp_dw = _products(proj_host, oracle.bf16_round(w)[None], oracle.bf16_round(g))
    assert relerr(out.cpu().numpy(), exp_out) < FWD_TOL
    assert relerr(out.cpu().numpy(), oracle.kpconv(*host, contraction="bf16")) < BF16_TOL
    assert relerr(out.cpu().numpy(), oracle.kpconv(*host)) < LOOSE_TOL
    grads = ops.kp_conv_grads(*args, t(g), proj=proj, contraction="bf16")
    exp_g = oracle.kpconv_grads(*host, g, contraction="bf16")
    assert relerr(grads[0].cpu().numpy(), exp_dw[0]) < GRAD_TOL
    for got, e, name in zip(grads, exp_g, ("dW", "dFeat", "dKernelPts", "dPts", "dSamples")):
        assert tuple(got.shape) == e.shape, name
        assert relerr(got.cpu().numpy(), e) < (BF16_TOL if name == "dW" else GRAD_TOL), name


def test_bf16_mode_rejects_unknown_names_and_wrong_projection(ops):
    pts, smp, nb, rng = _case(ops, 7, False)
    d = nb["dev"]
    kp, sigma = synthetic.kernel_points_sphere(1, 8)
    feats = t(rng.normal(size=(pts.shape[0], 8)).astype(np.float32))
    w = t(rng.normal(size=(64, 8)).astype(np.float32))
    args = (d["pts"], feats, d["samples"], d["neigh"], d["ends"], d["radii"], t(kp), sigma, w)
    with pytest.raises(RuntimeError):
        ops.kp_conv(*args, contraction="fp8")
    out, proj32 = ops.kp_conv(*args, return_proj=True)
    with pytest.raises(RuntimeError):                # an fp32 projection cannot feed the bf16 backward pass
        ops.kp_conv_grads(*args, torch.ones_like(out), proj=proj32, contraction="bf16")


def test_hierarchical_encoder_bf16(oracle):
    # Config 5 in small: room-style clouds normalised by their longest side, four Poisson-disk levels, each followed
    # by neighbor search, density and an MCConv (division by the density) with the contraction in bf16; forward and
    # backward through autograd, every level checked against the oracle fed with the same inputs.
    import pccnn_lib_amd as lib
    batch, num_pts = 2, 6000
    pts = np.concatenate([synthetic.room(50 + b, num_pts) / 10.0 for b in range(batch)]).astype(np.float32)
    ids = np.repeat(np.arange(batch, dtype=np.int32), num_pts)
    radii_levels = (0.025, 0.05, 0.1, 0.2)
    channels = (32, 64, 128, 256)
    rng = np.random.default_rng(11)
    torch.manual_seed(11)
    pc = lib.pc.Pointcloud(pts, ids, device=DEV)
    feats = t(rng.normal(size=(pts.shape[0], 8)).astype(np.float32)).requires_grad_(True)
    cur_pc, cur_feats, c_in = pc, feats, 8
    levels = []
    for radius, c_out in zip(radii_levels, channels):
        r3 = torch.full((3,), radius, device=DEV)
        pool = lib.pc.PointPooling(cur_pc, r3)
        out_pc = lib.pc.Pointcloud(pool.pool_tensor(cur_pc.pts_), pool.pool_tensor(cur_pc.batch_ids_))
        cur_pc.compute_pdf(np.full(3, 0.2 * radius, np.float32))
        layer = lib.pc.layers.MCConv(3, c_in, c_out, 8).to(DEV)
        layer.contraction_ = "bf16"
        out, nbh = layer(cur_pc, out_pc, cur_feats, 2.0 * radius)
        out.retain_grad()
        levels.append(dict(pc_in=cur_pc, pc_out=out_pc, layer=layer, feats=cur_feats, out=out, nbh=nbh,
                           radius=2.0 * radius, pool=pool))
        cur_pc, cur_feats, c_in = out_pc, torch.nn.functional.leaky_relu(out, 0.2), c_out
    assert levels[-1]["out"].shape[0] >= batch          # every cloud keeps at least one point
    g = rng.normal(size=tuple(levels[-1]["out"].shape)).astype(np.float32)
    levels[-1]["out"].backward(t(g))
    p = lambda x: x.detach().cpu().numpy()
    for lv in levels:
        pin, pout, layer = lv["pc_in"], lv["pc_out"], lv["layer"]
        hp, hi = p(pin.pts_), p(pin.batch_ids_)
        hs, hsi = p(pout.pts_), p(pout.batch_ids_)
        nb = oracle.neighborhood(hp, hi, hs, hsi, lv["radius"], batch_size=batch)
        assert np.array_equal(oracle.canonical_pairs(p(lv["nbh"].neighbors_)), oracle.canonical_pairs(nb["neighbors"]))
        radii = np.full(3, lv["radius"], np.float32)
        pdf = p(pin.pts_unnorm_pdf_ * torch.prod(t(radii)))
        host = (hp, pdf, p(lv["feats"]), hs, p(lv["nbh"].neighbors_), p(lv["nbh"].start_ids_), radii,
                p(layer.proj_axis_), p(layer.proj_bias_), p(layer.conv_weights_))
        assert relerr(p(lv["out"]), oracle.mcconv(*host, contraction="bf16")) < BF16_TOL
        exp_g = oracle.mcconv_grads(*host, p(lv["out"].grad), contraction="bf16")
        assert relerr(p(layer.conv_weights_.grad), exp_g[0]) < BF16_TOL
        assert relerr(p(layer.proj_axis_.grad), exp_g[2]) < BF16_TOL
    assert feats.grad is not None and bool(torch.isfinite(feats.grad).all())
