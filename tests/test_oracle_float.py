"""Pins the oracle's floating-point path (KDE, KPConv / MCConv forward and gradients) against the
formulations of the reference's own unit tests, float64 closed forms, special cases and torch
autograd.  CPU only."""
import numpy as np
import pytest
import torch

from pccnn_lib_amd import synthetic


def _cloud(models, batch, num_pts):
    pts = np.ascontiguousarray(models[:batch, :num_pts, :].reshape(-1, 3), np.float32)
    return pts, np.repeat(np.arange(batch, dtype=np.int32), num_pts)


# ------------------------------------------------------------------------------------ pdf

def test_pdf_matches_sklearn(oracle, models):
    # unit_test/test_pdf.py:52-60: sklearn KernelDensity per cloud, rtol = atol = 1e-2.
    from sklearn.neighbors import KernelDensity
    # bandwidth 0.025 as in unit_test/utest_pdf.ini Test_5 (the 300-neighbor cap is never reached).
    pts, ids = _cloud(models, 2, 1000)
    bw = 0.025
    _, pdf, nb = oracle.pointcloud_pdf(pts, ids, bw)
    assert np.diff(nb["ends"], prepend=0).max() < 300
    ref = []
    for b in range(2):
        kde = KernelDensity(bandwidth=bw).fit(pts[ids == b])
        ref.append(np.exp(kde.score_samples(pts[ids == b])))
    assert np.allclose(np.concatenate(ref), pdf, rtol=1e-2, atol=1e-2)


def test_pdf_closed_form_float64(oracle, models):
    pts, ids = _cloud(models, 2, 600)
    bw = np.array([0.05, 0.06, 0.07], np.float32)
    unnorm, _, nb = oracle.pointcloud_pdf(pts, ids, bw, manifold_dims=2)
    neigh, ends = nb["neighbors"], nb["ends"]
    ib = (np.float32(1.0) / bw).astype(np.float64)
    d = (pts[neigh[:, 0]].astype(np.float64) - pts[neigh[:, 1]].astype(np.float64)) * ib
    term = np.prod(ib) / (2.0 * 3.1415) ** (2 / 2.0) * np.exp(-0.5 * (d * d).sum(axis=1))
    expect = np.zeros(pts.shape[0])
    np.add.at(expect, neigh[:, 1], term)
    assert np.allclose(unnorm, expect, rtol=1e-5, atol=0)
    # the constant is 3.1415, not pi: with pi the result is off by more than the tolerance (m = 3)
    unnorm3 = oracle.compute_pdf(3, bw, pts, neigh, ends)
    with_pi = expect * (2.0 * 3.1415) / (2.0 * np.pi) ** 1.5
    assert not np.allclose(unnorm3, with_pi, rtol=1e-5, atol=0)


def test_pdf_isolated_point(oracle):
    pts = np.array([[0, 0, 0], [10, 10, 10]], np.float32)
    neigh = np.array([[0, 0], [1, 1]], np.int32)
    ends = np.array([1, 2], np.int32)
    bw = np.array([0.5, 0.25, 0.125], np.float32)
    out = oracle.compute_pdf(3, bw, pts, neigh, ends)
    assert np.allclose(out, 2 * 4 * 8 / (2 * 3.1415) ** 1.5, rtol=1e-6)


def test_pdf_grads_match_autograd(oracle, models):
    pts, ids = _cloud(models, 2, 300)
    bw = np.array([0.08, 0.08, 0.08], np.float32)
    _, _, nb = oracle.pointcloud_pdf(pts, ids, bw)
    neigh, ends = nb["neighbors"], nb["ends"]
    g = np.random.default_rng(0).normal(size=pts.shape[0]).astype(np.float32)
    got = oracle.compute_pdf_grads(3, bw, pts, neigh, ends, g)
    p = torch.tensor(pts, dtype=torch.float64, requires_grad=True)
    ib = torch.tensor((np.float32(1.0) / bw).astype(np.float64))
    d = (p[neigh[:, 0].astype(np.int64)] - p[neigh[:, 1].astype(np.int64)]) * ib
    term = torch.prod(ib) / (2.0 * 3.1415) ** 1.5 * torch.exp(-0.5 * (d * d).sum(dim=1))
    pdf = torch.zeros(pts.shape[0], dtype=torch.float64).index_add(0, torch.tensor(neigh[:, 1].astype(np.int64)), term)
    (pdf * torch.tensor(g, dtype=torch.float64)).sum().backward()
    # The op differentiates each pair term w.r.t. both of its end points (compute_pdf.cu:131-147).
    assert np.allclose(got, p.grad.numpy(), rtol=1e-4, atol=1e-4 * np.abs(p.grad.numpy()).max())


# ----------------------------------------------------------------------------------- conv

def _setup(oracle, models, radius, c_in, seed):
    pts, ids = _cloud(models, 2, 500)
    nb = oracle.neighborhood(pts, ids, pts, ids, radius)
    rng = np.random.default_rng(seed)
    feats = rng.uniform(0, 1, (pts.shape[0], c_in)).astype(np.float32)
    return pts, ids, nb, feats, rng


@pytest.mark.parametrize("k,c_in,c_out", [(16, 32, 24), (15, 8, 5)])
def test_kpconv_forward_matches_unit_test_numpy(oracle, models, k, c_in, c_out):
    # unit_test/test_kpconv.py:60-82
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.2, c_in, 33)
    kp, sigma = synthetic.kernel_points_sphere(1, k)
    w = rng.normal(0, np.sqrt(2.0 / (c_in * k)), (k * c_in, c_out)).astype(np.float32)
    radii = nb["radii"]
    neigh, ends = nb["neighbors"], nb["ends"]
    got = oracle.kpconv(pts, feats, pts, neigh, ends, radii, kp, sigma, w)
    diff = (pts[neigh[:, 0]] - pts[neigh[:, 1]]) / radii.reshape(1, -1)
    kd = np.linalg.norm(diff.reshape(-1, 1, 3) - kp.reshape(1, -1, 3), axis=-1) / sigma
    basis = np.clip(1.0 - kd, 0.0, 1.0)
    proj = np.zeros((pts.shape[0], c_in, k))
    for t in range(neigh.shape[0]):
        proj[neigh[t, 1]] += feats[neigh[t, 0]].reshape(-1, 1) * basis[t].reshape(1, -1)
    expect = proj.reshape(pts.shape[0], -1) @ w
    assert (basis > 0).mean() > 0.05          # the layout gives non-trivial weights
    assert np.allclose(expect, got, rtol=1e-4, atol=1e-4)
    assert np.allclose(expect, got, rtol=1e-5, atol=1e-5 * np.abs(expect).max())


def test_kpconv_single_neighbor_special_case(oracle):
    # one sample, one neighbor (itself), all-ones features: out = sum_k w_k * sum_f W[f*K+k]
    pts = np.array([[0.1, 0.2, 0.3]], np.float32)
    neigh, ends = np.array([[0, 0]], np.int32), np.array([1], np.int32)
    kp, sigma = synthetic.kernel_points_sphere(2, 8)
    w = np.random.default_rng(1).normal(size=(8 * 4, 3)).astype(np.float32)
    out = oracle.kpconv(pts, np.ones((1, 4), np.float32), pts, neigh, ends, np.full(3, 0.5, np.float32), kp, sigma, w)
    basis = np.clip(1.0 - np.linalg.norm(kp, axis=1) / sigma, 0, 1)       # diff = 0
    assert basis[0] == 1.0
    expect = (w.reshape(4, 8, 3) * basis.reshape(1, 8, 1)).sum(axis=(0, 1))
    assert np.allclose(out[0], expect, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("num_mlps", [1, 2])
def test_mcconv_forward_matches_unit_test_numpy(oracle, models, num_mlps):
    # unit_test/test_mcconv.py:65-91 (num_mlps = 1 there; 2 follows mcconv.cu:64-68)
    c_in, hidden, c_out = 32, 16, 12
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.2, c_in, 33)
    unnorm, _, _ = oracle.pointcloud_pdf(pts, ids, 0.05)
    radii = nb["radii"]
    pdf = (unnorm * np.prod(radii)).astype(np.float32)
    axis = rng.normal(0, np.sqrt(1 / 3), (3, hidden * num_mlps)).astype(np.float32)
    bias = rng.normal(0, 0.1, (1, hidden * num_mlps)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (c_in * hidden)), (num_mlps, hidden * c_in, c_out // num_mlps)).astype(np.float32)
    neigh, ends = nb["neighbors"], nb["ends"]
    got = oracle.mcconv(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, w)
    diff = (pts[neigh[:, 0]] - pts[neigh[:, 1]]) / radii.reshape(1, -1)
    proj_ax = np.dot(diff, axis) + bias
    proj_ax = np.where(proj_ax < 0, proj_ax * 0.2, proj_ax) / pdf[neigh[:, 0]].reshape(-1, 1)
    ktot = hidden * num_mlps
    proj = np.zeros((pts.shape[0], c_in, ktot))
    for t in range(neigh.shape[0]):
        proj[neigh[t, 1]] += feats[neigh[t, 0]].reshape(-1, 1) * proj_ax[t].reshape(1, -1)
    if num_mlps == 1:
        expect = proj.reshape(pts.shape[0], -1) @ w.reshape(c_in * hidden, -1)
    else:
        pr = proj.reshape(pts.shape[0], num_mlps, -1)
        expect = np.concatenate([pr[:, i, :] @ w[i] for i in range(num_mlps)], axis=1)
    assert np.allclose(expect, got, rtol=1e-4, atol=1e-4)
    assert np.allclose(expect, got, rtol=1e-5, atol=1e-5 * np.abs(expect).max())


def _torch_forward(kind, pts, samples, feats, neigh, ends, radii, basis_params, weights, num_mlps=1):
    """float64 torch restatement of the forward; autograd supplies the analytic gradients."""
    n_idx = torch.tensor(neigh[:, 0].astype(np.int64))
    s_idx = torch.tensor(neigh[:, 1].astype(np.int64))
    inv_r = torch.tensor((np.float32(1.0) / radii).astype(np.float64))
    diff = (pts[n_idx] - samples[s_idx]) * inv_r
    if kind == "kp":
        kp, sigma = basis_params
        dist = torch.sqrt(((kp[None] - diff[:, None, :]) ** 2).sum(-1))
        basis = torch.clamp(1.0 - dist / sigma, 0.0, 1.0)
    elif kind == "kpn":
        # kpconvn.cu:37-46; the reference gives the density no gradient, so it enters as a constant
        kp, sigma, pdf = basis_params
        dist = torch.sqrt(((kp[None] - diff[:, None, :]) ** 2).sum(-1))
        basis = torch.clamp(1.0 - dist / sigma, 0.0, 1.0) / pdf.detach()[n_idx][:, None]
    elif kind == "gauss":
        kp, sigma, pdf = basis_params
        d2 = ((kp[None] - diff[:, None, :]) ** 2).sum(-1)
        basis = torch.exp(-d2 / (2.0 * sigma * sigma)) / pdf[n_idx][:, None]
    elif kind == "explicit":
        basis = basis_params
    else:
        axis, bias, pdf = basis_params
        basis = torch.nn.functional.leaky_relu(diff @ axis + bias, 0.2) / pdf[n_idx][:, None]
    m = ends.shape[0]
    pair = feats[n_idx][:, :, None] * basis[:, None, :]
    proj = torch.zeros((m, feats.shape[1], basis.shape[1]), dtype=torch.float64).index_add(0, s_idx, pair)
    proj = proj.reshape(m, num_mlps, -1).transpose(0, 1)
    out = torch.matmul(proj, weights.reshape(num_mlps, proj.shape[2], -1))
    return out.transpose(0, 1).reshape(m, -1)


def _relerr(a, b):
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def test_kpconv_grads_match_autograd(oracle, models):
    c_in, c_out, k = 16, 10, 16
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.25, c_in, 7)
    # distinct sample set so that dPts and dSamples are separate tensors
    smp = (pts[::3] + rng.normal(0, 0.01, pts[::3].shape)).astype(np.float32)
    nb = oracle.neighborhood(pts, ids, smp, ids[::3], 0.25)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    kp, sigma = synthetic.kernel_points_sphere(3, k)
    w = rng.normal(0, 0.2, (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    got = oracle.kpconv_grads(pts, feats, smp, neigh, ends, radii, kp, sigma, w, g)
    tp, ts, tf, tkp, tw = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (pts, smp, feats, kp, w)]
    out = _torch_forward("kp", tp, ts, tf, neigh, ends, radii, (tkp, float(np.float32(sigma))), tw)
    (out * torch.tensor(g, dtype=torch.float64)).sum().backward()
    for mine, ref, name in zip(got, (tw, tf, tkp, tp, ts), ("dW", "dFeat", "dKp", "dPts", "dSamples")):
        assert _relerr(mine, ref.grad.numpy()) < 1e-4, name


def test_kpconv_grad_kink_follows_reference_formula(oracle):
    # A pair at distance 0 from the centre kernel point: the reference's gradient is exactly 0
    # there (kernel_pts_basis.cu:58-66: the (kp - d) factor vanishes), whatever autograd says.
    pts = np.array([[0.0, 0.0, 0.0]], np.float32)
    neigh, ends = np.array([[0, 0]], np.int32), np.array([1], np.int32)
    kp = np.zeros((1, 3), np.float32)
    out = oracle.kpconv_grads(pts, np.ones((1, 2), np.float32), pts, neigh, ends, np.ones(3, np.float32), kp, 0.5,
                              np.ones((2, 1), np.float32), np.ones((1, 1), np.float32))
    assert np.all(out[2] == 0) and np.all(out[3] == 0) and np.all(out[4] == 0)


@pytest.mark.parametrize("num_mlps", [1, 2])
def test_mcconv_grads_match_autograd(oracle, models, num_mlps):
    c_in, c_out, hidden = 8, 6, 8
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.25, c_in, 9)
    smp = (pts[::3] + rng.normal(0, 0.01, pts[::3].shape)).astype(np.float32)
    nb = oracle.neighborhood(pts, ids, smp, ids[::3], 0.25)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    axis = rng.normal(0, 0.6, (3, hidden * num_mlps)).astype(np.float32)
    bias = rng.normal(0, 0.2, (1, hidden * num_mlps)).astype(np.float32)
    w = rng.normal(0, 0.2, (num_mlps, hidden * c_in, c_out // num_mlps)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    got = oracle.mcconv_grads(pts, pdf, feats, smp, neigh, ends, radii, axis, bias, w, g)
    tp, tpdf, tf, ts, ta, tb, tw = [torch.tensor(a, dtype=torch.float64, requires_grad=True)
                                     for a in (pts, pdf, feats, smp, axis, bias, w)]
    out = _torch_forward("mlp", tp, ts, tf, neigh, ends, radii, (ta, tb, tpdf), tw, num_mlps)
    (out * torch.tensor(g, dtype=torch.float64)).sum().backward()
    names = ("dW", "dFeat", "dAxis", "dBias", "dPdf", "dPts", "dSamples")
    for mine, ref, name in zip(got, (tw, tf, ta, tb, tpdf, tp, ts), names):
        assert mine.shape == tuple(ref.shape), name
        assert _relerr(mine, ref.grad.numpy()) < 1e-4, name


def test_torch_cpu_step_matches_the_scalar_oracle(oracle, models):
    """The multi-threaded CPU baseline (padded, batched form) computes what the scalar oracle computes, including the
    samples whose list is shorter than the padding, an empty list and a ragged last chunk."""
    from oracle import torch_cpu
    c_in, c_out, hidden = 8, 6, 8
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.2, c_in, 21)
    pts[-1] += 50.0                                   # a point far from everything: its only neighbor is itself
    nb = oracle.neighborhood(pts, ids, pts, ids, 0.2)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    axis = rng.normal(0, 0.6, (3, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.2, (1, hidden)).astype(np.float32)
    w = rng.normal(0, 0.2, (1, hidden * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    out, grads = torch_cpu.mcconv_step(pts, pdf, feats, neigh, ends, radii, axis, bias, w, g, samples_per_chunk=300)
    ref = oracle.mcconv(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, w)
    dw, dfeat, daxis, dbias, dpdf, dpts, dsmp = oracle.mcconv_grads(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, w, g)
    assert _relerr(out, ref) < 1e-5
    for name, want in (("weights", dw), ("feats", dfeat), ("axis", daxis), ("bias", dbias), ("pdf", dpdf),
                       ("pts", dpts + dsmp)):
        assert _relerr(grads[name].reshape(want.shape), want) < 1e-4, name


def test_torch_cpu_kpconv_step_matches_the_scalar_oracle(oracle, models):
    """The multi-threaded CPU baseline of the KPConv step (weights, features and position gradients) against the
    scalar oracle, with an isolated point and a ragged last chunk."""
    from oracle import torch_cpu
    c_in, c_out = 6, 5
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.2, c_in, 23)
    pts[-1] += 50.0
    nb = oracle.neighborhood(pts, ids, pts, ids, 0.2)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    kp, sigma = synthetic.kernel_points_sphere(5, 15)
    w = rng.normal(0, 0.2, (15 * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    out, grads = torch_cpu.kpconv_step(pts, feats, neigh, ends, radii, kp, sigma, w, g, samples_per_chunk=300)
    ref = oracle.kpconv(pts, feats, pts, neigh, ends, radii, kp, sigma, w)
    dw, dfeat, _, dpts, dsmp = oracle.kpconv_grads(pts, feats, pts, neigh, ends, radii, kp, sigma, w, g)
    assert _relerr(out, ref) < 1e-5
    for name, want in (("weights", dw), ("feats", dfeat), ("pts", dpts + dsmp)):
        assert _relerr(grads[name].reshape(want.shape), want) < 1e-4, name


def test_weight_variance_equals_projection_norm(oracle, models):
    # The double sum over neighbor pairs of (w_i . w_j)(F_i . F_j) (compute_variance_weights.cu:38-108) is the
    # squared Frobenius norm of the sample's projection tile; the literal O(n^2) restatement must agree with it.
    pts, ids, nb, feats, rng = _setup(oracle, models, 0.2, 12, 3)
    kp, sigma = synthetic.kernel_points_sphere(4, 16)
    neigh, ends, radii = nb["neighbors"], nb["ends"], nb["radii"]
    basis, _ = oracle.conv_basis(oracle.KP, pts, pts, neigh, radii, kp, sigma=sigma)
    val, per = oracle.variance_weights(basis, feats, neigh, ends)
    proj = oracle.feat_basis_proj(basis, feats, neigh, ends).astype(np.float64)
    norms = (proj ** 2).sum(axis=(1, 2))
    assert np.allclose(per, norms, rtol=1e-5)
    assert np.isclose(val, 1.0 / norms.mean(), rtol=1e-5)
    assert np.isclose(oracle.kpconv_weight_var(pts, feats, pts, neigh, ends, radii, kp, sigma), val, rtol=1e-6)
    # one sample with a single neighbor: (w . w)(F . F)
    one = oracle.variance_weights(basis[:1], feats, neigh[:1], np.array([1], np.int32))[0]
    f0 = feats[neigh[0, 0]].astype(np.float64)
    assert np.isclose(1.0 / one, (basis[0].astype(np.float64) ** 2).sum() * (f0 ** 2).sum(), rtol=1e-6)


# ----------------------------------------------------- the other convolution families
#
# The reference ships no unit test for KPConvN, PCCNN, PointConv or SPHConv, so their restatements are pinned by
# float64 torch formulations of the forward (kpconvn.cu, pccnn.cu, pointconv.cu, sphconv.cu read as formulas),
# autograd for the gradients, and special cases.

def _two_sets(oracle, models, c_in, seed, radius=0.25):
    pts, ids, nb, feats, rng = _setup(oracle, models, radius, c_in, seed)
    smp = (pts[::3] + rng.normal(0, 0.01, pts[::3].shape)).astype(np.float32)
    nb = oracle.neighborhood(pts, ids, smp, ids[::3], radius)
    return pts, smp, feats, nb["neighbors"], nb["ends"], nb["radii"], rng


def test_kpconvn_matches_float64_and_autograd(oracle, models):
    c_in, c_out, k = 8, 6, 16
    pts, smp, feats, neigh, ends, radii, rng = _two_sets(oracle, models, c_in, 11)
    kp, sigma = synthetic.kernel_points_sphere(3, k)
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    w = rng.normal(0, 0.2, (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    tp, ts, tf, tkp, tw = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (pts, smp, feats, kp, w)]
    tpdf = torch.tensor(pdf, dtype=torch.float64)
    out = _torch_forward("kpn", tp, ts, tf, neigh, ends, radii, (tkp, float(np.float32(sigma)), tpdf), tw)
    got = oracle.kpconvn(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma, w)
    assert _relerr(got, out.detach().numpy()) < 1e-5
    # dividing by a constant density c scales the KPConv result by 1/c
    half = oracle.kpconvn(pts, np.full_like(pdf, 2.0), feats, smp, neigh, ends, radii, kp, sigma, w)
    assert _relerr(half, 0.5 * oracle.kpconv(pts, feats, smp, neigh, ends, radii, kp, sigma, w)) < 1e-6
    (out * torch.tensor(g, dtype=torch.float64)).sum().backward()
    grads = oracle.kpconvn_grads(pts, pdf, feats, smp, neigh, ends, radii, kp, sigma, w, g)
    for mine, ref, name in zip(grads, (tw, tf, tkp, tp, ts), ("dW", "dFeat", "dKp", "dPts", "dSamples")):
        assert _relerr(mine, ref.grad.numpy()) < 1e-4, name


def test_pccnn_matches_float64_and_autograd(oracle, models):
    c_in, c_out, k = 8, 6, 16
    pts, smp, feats, neigh, ends, radii, rng = _two_sets(oracle, models, c_in, 12)
    kp, _ = synthetic.kernel_points_sphere(5, k)
    sigma = 0.4
    pdf = rng.uniform(0.5, 2.0, pts.shape[0]).astype(np.float32)
    w = rng.normal(0, 0.2, (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    tp, tpdf, ts, tf, tkp, tw = [torch.tensor(a, dtype=torch.float64, requires_grad=True)
                                 for a in (pts, pdf, smp, feats, kp, w)]
    out = _torch_forward("gauss", tp, ts, tf, neigh, ends, radii, (tkp, float(np.float32(sigma)), tpdf), tw)
    got = oracle.pccnn(pts, feats, pdf, smp, neigh, ends, radii, kp, sigma, w)
    assert _relerr(got, out.detach().numpy()) < 1e-5
    (out * torch.tensor(g, dtype=torch.float64)).sum().backward()
    grads = oracle.pccnn_grads(pts, feats, pdf, smp, neigh, ends, radii, kp, sigma, w, g)
    names = ("dW", "dFeat", "dKp", "dPdf", "dPts", "dSamples")
    for mine, ref, name in zip(grads, (tw, tf, tkp, tpdf, tp, ts), names):
        assert mine.shape == tuple(ref.shape), name
        assert _relerr(mine, ref.grad.numpy()) < 1e-4, name
    # a pair sitting on a kernel point has basis exactly 1 / pdf
    one = oracle.gauss_basis(np.zeros((1, 3), np.float32), np.array([4.0], np.float32), np.zeros((1, 3), np.float32),
                             np.array([[0, 0]], np.int32), np.ones(3, np.float32), np.zeros((1, 3), np.float32), 0.3)[0]
    assert one[0, 0] == 0.25


def test_pointconv_matches_float64_and_autograd(oracle, models):
    c_in, c_out, k = 8, 6, 16
    pts, smp, feats, neigh, ends, radii, rng = _two_sets(oracle, models, c_in, 13)
    axis = rng.normal(0, 0.6, (3, k)).astype(np.float32)
    bias = rng.normal(0, 0.2, (1, k)).astype(np.float32)
    w = rng.normal(0, 0.2, (k * c_in, c_out)).astype(np.float32)
    t = neigh.shape[0]
    n_idx, s_idx = neigh[:, 0].astype(np.int64), neigh[:, 1].astype(np.int64)
    # basis op (pointconv.cu:17-32) and its gradients
    tp, ts, ta, tb = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (pts, smp, axis, bias)]
    inv_r = torch.tensor((np.float32(1.0) / radii).astype(np.float64))
    tbasis = ((tp[n_idx] - ts[s_idx]) * inv_r) @ ta + tb
    basis, _ = oracle.pointconv_basis(pts, radii, smp, neigh, axis, bias)
    assert basis.shape == (t, k) and _relerr(basis, tbasis.detach().numpy()) < 1e-6
    gb = rng.normal(size=(t, k)).astype(np.float32)
    (tbasis * torch.tensor(gb, dtype=torch.float64)).sum().backward()
    grads = oracle.pointconv_basis_grads(pts, radii, smp, neigh, axis, bias, gb)
    for mine, ref, name in zip(grads, (tp, ts, ta, tb), ("dPts", "dSamples", "dAxis", "dBias")):
        assert mine.shape == tuple(ref.shape), name
        assert _relerr(mine, ref.grad.numpy()) < 1e-4, name
    # conv op with explicit basis values (pointconv.cu:61-101)
    act = np.maximum(basis, 0).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    tact, tf, tw = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (act, feats, w)]
    out = _torch_forward("explicit", tp.detach(), ts.detach(), tf, neigh, ends, radii, tact, tw)
    assert _relerr(oracle.pointconv(act, feats, neigh, ends, w), out.detach().numpy()) < 1e-5
    (out * torch.tensor(g, dtype=torch.float64)).sum().backward()
    for mine, ref, name in zip(oracle.pointconv_grads(act, feats, neigh, ends, w, g), (tw, tf, tact),
                               ("dW", "dFeat", "dBasis")):
        assert _relerr(mine, ref.grad.numpy()) < 1e-4, name
    proj = oracle.feat_basis_proj(act, feats, neigh, ends).astype(np.float64)
    assert np.isclose(oracle.pointconv_weight_var(act, feats, neigh, ends), 1.0 / (proj ** 2).sum(axis=(1, 2)).mean(),
                      rtol=1e-5)


def test_spherical_basis_bins(oracle):
    # Hand-placed offsets (radius 1): the bin of each is fixed by spherical_basis.cu:36-63.
    radial = np.array([0.5, 1.0], np.float32)
    azimuth = np.array([0.0, np.pi / 2], np.float32)          # atan() lies in (-pi/2, pi/2)
    polar = np.array([np.pi / 2, np.pi], np.float32)
    offs = np.array([[0.0, 0.0, 0.0],        # centre -> bin 0
                     [0.3, 0.1, 0.1],        # r<0.5, azimuth>0, polar<pi/2 -> (0,1,0)
                     [0.3, -0.1, -0.1],      # r<0.5, azimuth<0, polar>pi/2 -> (0,0,1)
                     [0.6, 0.5, 0.2],        # 0.5<r<1 -> (1,1,0)
                     [2.0, -1.0, -1.0]],     # r>1 clamps to the last radial bin -> (1,0,1)
                    np.float32)
    pts = offs
    smp = np.zeros((1, 3), np.float32)
    neigh = np.stack([np.arange(5), np.zeros(5)], axis=1).astype(np.int32)
    basis = oracle.spherical_basis(pts, smp, neigh, np.ones(3, np.float32), radial, azimuth, polar)
    assert basis.shape == (5, 9) and np.all(basis.sum(axis=1) == 1)
    expect = [0, 1 + (0 * 2 + 1) * 2 + 0, 1 + (0 * 2 + 0) * 2 + 1, 1 + (1 * 2 + 1) * 2 + 0, 1 + (1 * 2 + 0) * 2 + 1]
    assert list(basis.argmax(axis=1)) == expect


def test_sphconv_matches_float64_and_autograd(oracle, models):
    c_in, c_out = 8, 6
    pts, smp, feats, neigh, ends, radii, rng = _two_sets(oracle, models, c_in, 14)
    radial = np.array([0.4, 0.7, 1.0], np.float32)
    azimuth = np.linspace(-np.pi / 2, np.pi / 2, 5)[1:].astype(np.float32)
    polar = np.linspace(0, np.pi, 4)[1:].astype(np.float32)
    k = 3 * 4 * 3 + 1
    w = rng.normal(0, 0.2, (k * c_in, c_out)).astype(np.float32)
    g = rng.normal(size=(smp.shape[0], c_out)).astype(np.float32)
    basis = oracle.spherical_basis(pts, smp, neigh, radii, radial, azimuth, polar)
    assert basis.shape[1] == k and len(np.unique(basis.argmax(axis=1))) > 20
    cnt = np.diff(ends, prepend=0).astype(np.float64)
    tf, tw = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (feats, w)]
    out = _torch_forward("explicit", torch.tensor(pts, dtype=torch.float64), torch.tensor(smp, dtype=torch.float64), tf,
                         neigh, ends, radii, torch.tensor(basis, dtype=torch.float64), tw)
    out = out / (torch.tensor(cnt)[:, None] + 1e-6)
    got = oracle.sphconv(pts, feats, smp, neigh, ends, radii, radial, azimuth, polar, w)
    assert _relerr(got, out.detach().numpy()) < 1e-5
    (out * torch.tensor(g, dtype=torch.float64)).sum().backward()
    grads = oracle.sphconv_grads(pts, feats, smp, neigh, ends, radii, radial, azimuth, polar, w, g)
    assert _relerr(grads[0], tw.grad.numpy()) < 1e-4 and _relerr(grads[1], tf.grad.numpy()) < 1e-4
    # weight variance: mean over samples of |projection tile|^2 / count^2 (compute_variance_weights.cu:31-63)
    proj = oracle.feat_basis_proj(basis, feats, neigh, ends).astype(np.float64)
    per = np.where(cnt > 0, (proj ** 2).sum(axis=(1, 2)) / np.maximum(cnt, 1) ** 2, 0.0)
    val = oracle.sphconv_weight_var(pts, feats, smp, neigh, ends, radii, radial, azimuth, polar)
    assert np.isclose(val, 1.0 / per.mean(), rtol=1e-5)
