"""numpy front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Integer / per-pair arithmetic lives in ``pccnn_oracle.c`` (loaded through
ctypes); the dense contractions and the basis gradients, which the reference
expresses as ATen call sequences, are restated here in numpy.  Nothing in the
product package imports this module: only ``tests/``, the smoke check and the
benchmark's CPU-baseline leg do.

Reference citations are paths inside the reference repository.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile ``liboracle.so`` with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_store_neighbors.restype = ctypes.c_int64
        _lib.orc_brute_force_neighbors.restype = ctypes.c_int64
        _lib.orc_poisson_disk.restype = ctypes.c_int64
        _lib.orc_variance_weights.restype = ctypes.c_double
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


I64 = ctypes.c_int64
I32 = ctypes.c_int
F32 = ctypes.c_float

# --------------------------------------------------------------- host glue


def bounding_box(pts, batch_ids, batch_size):
    """pccnn_lib/pc/BoundingBox.py:17-18: per-cloud min - 1e-6 and max + 1e-6
    (fp32 adds of the fp32-rounded constant)."""
    pts = _f32(pts)
    d = pts.shape[1]
    mn = np.full((batch_size, d), np.inf, np.float32)
    mx = np.full((batch_size, d), -np.inf, np.float32)
    np.minimum.at(mn, batch_ids, pts)
    np.maximum.at(mx, batch_ids, pts)
    eps = np.float32(1e-6)
    return (mn - eps).astype(np.float32), (mx + eps).astype(np.float32)


def num_cells(aabb_min, aabb_max, cell_size):
    """pccnn_lib/pc/Grid.py:26-28: max over clouds of int32((max-min)/cell) + 1
    (fp32 division, truncation toward zero)."""
    q = (_f32(aabb_max) - _f32(aabb_min)) / _f32(cell_size)
    return (q.astype(np.int32) + 1).max(axis=0).astype(np.int32)


# ------------------------------------------------------------ index ops


def compute_keys(pts, batch_ids, aabb_min, ncells, cell_size):
    pts, batch_ids, aabb_min = _f32(pts), _i32(batch_ids), _f32(aabb_min)
    ncells, cell_size = _i32(ncells), _f32(cell_size)
    n, d = pts.shape
    out = np.empty(n, np.int64)
    rc = lib().orc_compute_keys(_p(pts), _p(batch_ids), _p(aabb_min), _p(ncells), _p(cell_size),
                                I64(n), I32(d), _p(out))
    assert rc == 0
    return out


def argsort_keys(keys):
    keys = _i64(keys)
    perm = np.empty(keys.shape[0], np.int32)
    assert lib().orc_argsort_keys(_p(keys), I64(keys.shape[0]), _p(perm)) == 0
    return perm


def build_grid_ds(sorted_keys, ncells, batch_size):
    sorted_keys, ncells = _i64(sorted_keys), _i32(ncells)
    pillars = int(batch_size) * int(ncells[0]) * int(ncells[1])
    ds = np.empty((pillars, 2), np.int32)
    rc = lib().orc_build_grid_ds(_p(sorted_keys), I64(sorted_keys.shape[0]), _p(ncells),
                                 I32(ncells.shape[0]), I64(pillars), _p(ds))
    assert rc == 0, rc
    return ds.reshape(int(batch_size), int(ncells[0]), int(ncells[1]), 2)


def offsets(d):
    out = np.zeros((243, d), np.int32)
    n = lib().orc_offsets(I32(d), _p(out))
    return out[:n].copy()


def find_ranges(sample_keys, pt_keys_sorted, grid_ds, ncells):
    sample_keys, pt_keys_sorted = _i64(sample_keys), _i64(pt_keys_sorted)
    grid_ds, ncells = _i32(grid_ds), _i32(ncells)
    d = ncells.shape[0]
    n_off = offsets(d).shape[0]
    m = sample_keys.shape[0]
    ranges = np.empty((m, n_off, 2), np.int32)
    got = lib().orc_find_ranges(_p(sample_keys), I64(m), _p(pt_keys_sorted), I64(pt_keys_sorted.shape[0]),
                                _p(grid_ds), _p(ncells), I32(d), _p(ranges))
    assert got == n_off
    return ranges


def find_neighbors(pts_sorted, pt_keys_sorted, samples, sample_keys, grid_ds, ncells, radii, max_neighbors=0):
    """pccnn_lib_ops/find_neighbors/find_neighbors.cu:27-66.
    Returns (neigh int32[T,2] = (sorted point index, sample index), ends int32[M])."""
    pts_sorted, samples, radii = _f32(pts_sorted), _f32(samples), _f32(radii)
    m, d = samples.shape
    ranges = find_ranges(sample_keys, pt_keys_sorted, grid_ds, ncells)
    n_off = ranges.shape[1]
    counts = np.empty(m, np.int32)
    lib().orc_count_neighbors(_p(samples), I64(m), _p(pts_sorted), _p(ranges), I32(n_off), _p(radii), I32(d),
                              _p(counts))
    ends = np.empty(m, np.int32)
    total = lib().orc_store_neighbors(_p(samples), I64(m), _p(pts_sorted), _p(ranges), I32(n_off), _p(radii),
                                      I32(d), _p(counts), I32(max_neighbors), None, _p(ends))
    neigh = np.empty((total, 2), np.int32)
    lib().orc_store_neighbors(_p(samples), I64(m), _p(pts_sorted), _p(ranges), I32(n_off), _p(radii),
                              I32(d), _p(counts), I32(max_neighbors), _p(neigh), _p(ends))
    return neigh, ends


def brute_force_neighbors(samples, sample_batch, pts, pt_batch, radii):
    samples, pts, radii = _f32(samples), _f32(pts), _f32(radii)
    sample_batch, pt_batch = _i32(sample_batch), _i32(pt_batch)
    m, d = samples.shape
    n = pts.shape[0]
    ends = np.empty(m, np.int32)
    total = lib().orc_brute_force_neighbors(_p(samples), _p(sample_batch), I64(m), _p(pts), _p(pt_batch), I64(n),
                                            _p(radii), I32(d), None, _p(ends))
    neigh = np.empty((total, 2), np.int32)
    lib().orc_brute_force_neighbors(_p(samples), _p(sample_batch), I64(m), _p(pts), _p(pt_batch), I64(n),
                                    _p(radii), I32(d), _p(neigh), _p(ends))
    return neigh, ends


def neighborhood(pts, batch_ids, samples, sample_batch_ids, radius, batch_size=None, max_neighbors=0):
    """The composition of pccnn_lib/pc/{BoundingBox,Grid,Neighborhood}.py
    (layers/KPConv.py:142-146): returns a dict with every intermediate and
    neighbors remapped to original point ids (Neighborhood.py:47-53)."""
    pts, samples = _f32(pts), _f32(samples)
    batch_ids, sample_batch_ids = _i32(batch_ids), _i32(sample_batch_ids)
    d = pts.shape[1]
    radii = np.broadcast_to(_f32(radius), (d,)).copy()
    if batch_size is None:
        batch_size = int(batch_ids.max()) + 1
    mn, mx = bounding_box(pts, batch_ids, batch_size)
    nc = num_cells(mn, mx, radii)
    keys = compute_keys(pts, batch_ids, mn, nc, radii)
    perm = argsort_keys(keys)
    skeys = keys[perm]
    spts = pts[perm]
    ds = build_grid_ds(skeys, nc, batch_size)
    sample_keys = compute_keys(samples, sample_batch_ids, mn, nc, radii)
    neigh_sorted, ends = find_neighbors(spts, skeys, samples, sample_keys, ds, nc, radii, max_neighbors)
    neigh = neigh_sorted.copy()
    neigh[:, 0] = perm[neigh_sorted[:, 0]]
    return dict(aabb_min=mn, aabb_max=mx, num_cells=nc, keys=keys, perm=perm, sorted_keys=skeys,
                sorted_pts=spts, grid_ds=ds, sample_keys=sample_keys, neigh_sorted=neigh_sorted,
                neighbors=neigh, ends=ends, radii=radii)


def canonical_pairs(neigh):
    """Sort pairs by (sample, neighbor id): the order-free form used to compare neighbor lists."""
    neigh = np.asarray(neigh)
    order = np.lexsort((neigh[:, 0], neigh[:, 1]))
    return neigh[order]


# ------------------------------------------------------------------ pdf


def compute_pdf(manifold_dims, bandwidth, pts, neigh, ends):
    pts, bandwidth, neigh, ends = _f32(pts), _f32(bandwidth), _i32(neigh), _i32(ends)
    n, d = pts.shape
    out = np.empty(n, np.float32)
    lib().orc_compute_pdf(I32(manifold_dims), _p(bandwidth), _p(pts), I64(n), I32(d), _p(neigh), _p(ends), _p(out))
    return out


def compute_pdf_grads(manifold_dims, bandwidth, pts, neigh, ends, in_grads):
    pts, bandwidth, neigh, ends, in_grads = _f32(pts), _f32(bandwidth), _i32(neigh), _i32(ends), _f32(in_grads)
    n, d = pts.shape
    out = np.empty((n, d), np.float32)
    lib().orc_compute_pdf_grads(I32(manifold_dims), _p(bandwidth), _p(pts), I64(n), I32(d), _p(neigh), _p(ends),
                                _p(in_grads), _p(out))
    return out


def pointcloud_pdf(pts, batch_ids, bandwidth, manifold_dims=None):
    """pccnn_lib/pc/Pointcloud.py:81-109: search radius 4*bandwidth, cap 300, KDE, then the
    per-cloud normalisation.  Returns (unnormalised pdf, normalised pdf, neighborhood dict)."""
    pts, batch_ids = _f32(pts), _i32(batch_ids)
    d = pts.shape[1]
    bw = np.broadcast_to(_f32(bandwidth), (d,)).copy()
    radii = (bw * np.float32(4.0)).astype(np.float32)
    nb = neighborhood(pts, batch_ids, pts, batch_ids, radii, max_neighbors=300)
    m = d if manifold_dims is None else manifold_dims
    unnorm = compute_pdf(m, bw, pts, nb["neighbors"], nb["ends"])
    counts = np.bincount(batch_ids).astype(np.int32)
    return unnorm, (unnorm / counts[batch_ids].astype(np.float32)).astype(np.float32), nb


# -------------------------------------------------------------- pooling


def poisson_disk_sampling(sorted_keys, neigh, ends, ncells):
    sorted_keys, neigh, ends, ncells = _i64(sorted_keys), _i32(neigh), _i32(ends), _i32(ncells)
    n = sorted_keys.shape[0]
    used = np.empty(n, np.int32)
    lib().orc_poisson_disk(_p(sorted_keys), I64(n), _p(neigh), _p(ends), _p(ncells), I32(ncells.shape[0]), _p(used))
    return np.nonzero(used)[0].astype(np.int64).reshape(-1, 1)


# ----------------------------------------------------------------- conv

KP, MLP = 0, 1


def conv_basis(kind, pts, samples, neigh, radii, kp_or_axis, bias=None, sigma=1.0, pdf=None):
    pts, samples, neigh, radii, kp_or_axis = _f32(pts), _f32(samples), _i32(neigh), _f32(radii), _f32(kp_or_axis)
    t = neigh.shape[0]
    d = pts.shape[1]
    k = kp_or_axis.shape[0] if kind == KP else kp_or_axis.shape[1]
    bias = _f32(bias).reshape(-1) if bias is not None else None
    pdf = _f32(pdf) if pdf is not None else None
    basis = np.empty((t, k), np.float32)
    diff = np.empty((t, d), np.float32)
    lib().orc_conv_basis(I32(kind), _p(pts), _p(samples), _p(neigh), I64(t), _p(radii), I32(d), I32(k),
                         _p(kp_or_axis), _p(bias), F32(sigma), _p(pdf), _p(basis), _p(diff))
    return basis, diff


def feat_basis_proj(basis, feats, neigh, ends):
    basis, feats, neigh, ends = _f32(basis), _f32(feats), _i32(neigh), _i32(ends)
    m = ends.shape[0]
    c_in, k = feats.shape[1], basis.shape[1]
    out = np.empty((m, c_in, k), np.float32)
    lib().orc_feat_basis_proj(_p(basis), _p(feats), _p(neigh), _p(ends), I64(m), I32(c_in), I32(k), _p(out))
    return out


def feat_basis_proj_grads(basis, feats, neigh, ends, proj_grads):
    basis, feats, neigh, ends = _f32(basis), _f32(feats), _i32(neigh), _i32(ends)
    proj_grads = _f32(proj_grads)
    m = ends.shape[0]
    n, c_in = feats.shape
    k = basis.shape[1]
    fg = np.empty((n, c_in), np.float32)
    bg = np.empty((neigh.shape[0], k), np.float32)
    lib().orc_feat_basis_proj_grads(_p(basis), _p(feats), _p(neigh), _p(ends), I64(m), I64(n), I32(c_in), I32(k),
                                    _p(proj_grads), _p(fg), _p(bg))
    return fg, bg


def _pt_diff_grads(n, m, neigh, radii, diff_grads):
    """pccnn_lib_ops/pcconvs/shared/pt_diff.cu:51-80."""
    g = diff_grads.astype(np.float64) * (np.float32(1.0) / _f32(radii)).astype(np.float64)
    d = g.shape[1]
    dp = np.zeros((n, d), np.float64)
    dsm = np.zeros((m, d), np.float64)
    np.add.at(dp, neigh[:, 0], g)
    np.add.at(dsm, neigh[:, 1], g)
    return dp.astype(np.float32), (-dsm).astype(np.float32)


def bf16_round(a):
    """fp32 -> nearest bf16 (ties to even) -> fp32.  The reference has no bf16 mode; this is the operand rounding
    of the bf16 contraction of config 5 ("features bf16 for the MFMA contraction with fp32 accumulation")."""
    a = _f32(a)
    u = a.view(np.uint32).astype(np.uint64)
    r = (((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)
    return np.where(np.isnan(a), a, r).astype(np.float32)


def _operands(contraction):
    if contraction == "f32":
        return lambda x: x
    if contraction == "bf16":
        return bf16_round
    raise ValueError("contraction must be 'f32' or 'bf16'")


def kpconv(pts, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, contraction="f32"):
    """pccnn_lib_ops/pcconvs/kpconv.cu:32-60.  contraction="bf16": both operands of the matmul rounded to bf16."""
    rnd = _operands(contraction)
    basis, _ = conv_basis(KP, pts, samples, neigh, radii, kernel_pts, sigma=sigma)
    proj = feat_basis_proj(basis, feats, neigh, ends)
    m = ends.shape[0]
    out = rnd(proj.reshape(m, -1)).astype(np.float64) @ rnd(_f32(weights)).astype(np.float64)
    return out.astype(np.float32)


def kpconv_grads(pts, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, in_grads, contraction="f32"):
    """pccnn_lib_ops/pcconvs/kpconv.cu:63-112 with kernel_pts_basis.cu:41-70.
    Returns [dW, dFeat, dKernelPts, dPts, dSamples].  contraction="bf16": the operands of both matmuls (projection,
    weights, incoming gradients) rounded to bf16."""
    rnd = _operands(contraction)
    pts, samples, neigh, kernel_pts = _f32(pts), _f32(samples), _i32(neigh), _f32(kernel_pts)
    weights, in_grads = _f32(weights), _f32(in_grads)
    m = ends.shape[0]
    basis, diff = conv_basis(KP, pts, samples, neigh, radii, kernel_pts, sigma=sigma)
    proj = feat_basis_proj(basis, feats, neigh, ends).reshape(m, -1)
    dw = (rnd(proj).astype(np.float64).T @ rnd(in_grads).astype(np.float64)).astype(np.float32)
    dproj = (rnd(in_grads).astype(np.float64) @ rnd(weights).astype(np.float64).T).astype(np.float32)
    dfeat, dbasis = feat_basis_proj_grads(basis, feats, neigh, ends, dproj)
    # kernel_pts_basis_grads: fp32 distances and mask as the reference forms them.
    sig = np.float32(sigma)
    diff_kp = kernel_pts[None, :, :] - diff[:, None, :]                      # [T,K,D] fp32
    sq = diff_kp * diff_kp
    dist = sq[..., 0]
    for i in range(1, sq.shape[-1]):
        dist = dist + sq[..., i]
    dist = np.sqrt(np.maximum(dist, np.float32(0.0)))
    result = np.float32(1.0) - dist / sig
    inv_dist = (np.float32(1.0) / (dist + np.float32(1e-6))).astype(np.float64)
    mask = (result >= 0.0).astype(np.float64)
    cur = -(dbasis.astype(np.float64) * mask) / np.float64(sig)
    cur = cur[..., None] * inv_dist[..., None] * diff_kp.astype(np.float64)  # [T,K,D]
    ddiff = -cur.sum(axis=1)
    dkp = cur.sum(axis=0).astype(np.float32)
    dpts, dsamples = _pt_diff_grads(pts.shape[0], samples.shape[0], neigh, radii, ddiff)
    return [dw, dfeat, dkp, dpts, dsamples]


def mcconv(pts, pdf, feats, samples, neigh, ends, radii, axis, bias, weights, contraction="f32"):
    """pccnn_lib_ops/pcconvs/mcconv.cu:32-71 (weights [numMLPs, H*Cin/.., Cout/numMLPs]).  contraction as in kpconv."""
    rnd = _operands(contraction)
    weights = _f32(weights)
    num_mlps = weights.shape[0]
    basis, _ = conv_basis(MLP, pts, samples, neigh, radii, axis, bias=bias, pdf=pdf)
    proj = feat_basis_proj(basis, feats, neigh, ends)
    m = ends.shape[0]
    proj = rnd(proj).reshape(m, num_mlps, -1).transpose(1, 0, 2).astype(np.float64)
    out = np.matmul(proj, rnd(weights).astype(np.float64))                   # [mlps, M, Cout/mlps]
    return out.transpose(1, 0, 2).reshape(m, -1).astype(np.float32)


def mcconv_grads(pts, pdf, feats, samples, neigh, ends, radii, axis, bias, weights, in_grads, contraction="f32"):
    """pccnn_lib_ops/pcconvs/mcconv.cu:73-143 with mlp_basis.cu:50-96.
    Returns [dW, dFeat, dAxis, dBias, dPdf, dPts, dSamples].  contraction as in kpconv_grads."""
    rnd = _operands(contraction)
    pts, samples, neigh, axis = _f32(pts), _f32(samples), _i32(neigh), _f32(axis)
    weights, in_grads, pdf = _f32(weights), _f32(in_grads), _f32(pdf)
    bias = _f32(bias).reshape(1, -1)
    num_mlps = weights.shape[0]
    m = ends.shape[0]
    g = rnd(in_grads).reshape(m, num_mlps, -1).transpose(1, 0, 2).astype(np.float64)
    basis, diff = conv_basis(MLP, pts, samples, neigh, radii, axis, bias=bias, pdf=pdf)
    proj = feat_basis_proj(basis, feats, neigh, ends)
    projr = rnd(proj).reshape(m, num_mlps, -1).transpose(1, 0, 2).astype(np.float64)
    dw = np.matmul(projr.transpose(0, 2, 1), g).astype(np.float32)
    dproj = np.matmul(g, rnd(weights).astype(np.float64).transpose(0, 2, 1))
    dproj = dproj.transpose(1, 0, 2).reshape(m, -1).astype(np.float32)
    dfeat, dbasis = feat_basis_proj_grads(basis, feats, neigh, ends, dproj)
    # mlp_basis_grads (pDiv = true): activations in fp32 as the forward forms them.
    npdf = pdf[neigh[:, 0]]
    act = diff[:, 0:1] * axis[0:1, :]
    for i in range(1, diff.shape[1]):
        act = act + diff[:, i:i + 1] * axis[i:i + 1, :]
    act = act + bias
    act = np.where(act > 0, act, act * np.float32(0.2)).astype(np.float32)
    act64, db64, npdf64 = act.astype(np.float64), dbasis.astype(np.float64), npdf.astype(np.float64)
    dpdf_pair = ((-1.0 * act64 * db64) / (npdf64 * npdf64)[:, None]).sum(axis=1)
    cur = db64 / npdf64[:, None]
    cur = cur * np.where(act > 0, 1.0, 0.2)
    dbias = cur.sum(axis=0, keepdims=True).astype(np.float32)
    ddiff = cur @ axis.astype(np.float64).T
    daxis = (diff.astype(np.float64).T @ cur).astype(np.float32)
    dpdf = np.zeros(pdf.shape[0], np.float64)
    np.add.at(dpdf, neigh[:, 0], dpdf_pair)
    dpts, dsamples = _pt_diff_grads(pts.shape[0], samples.shape[0], neigh, radii, ddiff)
    return [dw, dfeat, daxis, dbias, dpdf.astype(np.float32), dpts, dsamples]


def variance_weights(basis, feats, neigh, ends):
    """compute_variance_weights.cu:114-170 (no division by the neighbor count).  Returns (1 / mean, per-sample sums)."""
    basis, feats, neigh, ends = _f32(basis), _f32(feats), _i32(neigh), _i32(ends)
    m = ends.shape[0]
    per = np.empty(m, np.float64)
    val = lib().orc_variance_weights(_p(basis), _p(feats), _p(neigh), _p(ends), I64(m), I32(feats.shape[1]),
                                     I32(basis.shape[1]), _p(per))
    return np.float32(val), per


def kpconv_weight_var(pts, feats, samples, neigh, ends, radii, kernel_pts, sigma):
    """pccnn_lib_ops/pcconvs/kpconv.cu:115-136."""
    basis, _ = conv_basis(KP, pts, samples, neigh, radii, kernel_pts, sigma=sigma)
    return variance_weights(basis, feats, neigh, ends)[0]


def mcconv_weight_var(pts, pdf, feats, samples, neigh, ends, radii, axis, bias):
    """pccnn_lib_ops/pcconvs/mcconv.cu:145-172."""
    basis, _ = conv_basis(MLP, pts, samples, neigh, radii, axis, bias=bias, pdf=pdf)
    return variance_weights(basis, feats, neigh, ends)[0]


# ------------------------------------------------ the other convolution families
#
# They reuse the pair offsets and the KPConv basis of orc_conv_basis and the projection / projection-gradient
# routines above; what differs per family is restated here in numpy, fp32 where the reference computes in fp32
# (the basis values), float64 for the sums the tolerance leaves open.


def _dense(proj, weights):
    m = proj.shape[0]
    return (proj.reshape(m, -1).astype(np.float64) @ _f32(weights).astype(np.float64)).astype(np.float32)


def _dense_grads(proj, weights, in_grads):
    m = proj.shape[0]
    g = _f32(in_grads).astype(np.float64)
    dw = (proj.reshape(m, -1).astype(np.float64).T @ g).astype(np.float32)
    dproj = (g @ _f32(weights).astype(np.float64).T).astype(np.float32)
    return dw, dproj


def _kp_basis_grads(diff, kernel_pts, sigma, dbasis):
    """kernel_pts_basis.cu:41-70 -> (dDiff [T,D] float64, dKernelPts [K,D] float32)."""
    sig = np.float32(sigma)
    diff_kp = kernel_pts[None, :, :] - diff[:, None, :]
    sq = diff_kp * diff_kp
    dist = sq[..., 0]
    for i in range(1, sq.shape[-1]):
        dist = dist + sq[..., i]
    dist = np.sqrt(np.maximum(dist, np.float32(0.0)))
    result = np.float32(1.0) - dist / sig
    inv_dist = (np.float32(1.0) / (dist + np.float32(1e-6))).astype(np.float64)
    mask = (result >= 0.0).astype(np.float64)
    cur = -(dbasis.astype(np.float64) * mask) / np.float64(sig)
    cur = cur[..., None] * inv_dist[..., None] * diff_kp.astype(np.float64)
    return -cur.sum(axis=1), cur.sum(axis=0).astype(np.float32)


def kpconvn_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma):
    """kpconvn.cu:37-46: the KPConv correlation divided (fp32) by the density of the neighbor."""
    basis, diff = conv_basis(KP, pts, samples, neigh, radii, kernel_pts, sigma=sigma)
    npdf = _f32(pdf)[_i32(neigh)[:, 0]].reshape(-1, 1)
    return (basis / npdf).astype(np.float32), diff, npdf


def kpconvn(pts, pdf, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights):
    """pccnn_lib_ops/pcconvs/kpconvn.cu:25-58."""
    basis, _, _ = kpconvn_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma)
    return _dense(feat_basis_proj(basis, feats, neigh, ends), weights)


def kpconvn_grads(pts, pdf, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, in_grads):
    """pccnn_lib_ops/pcconvs/kpconvn.cu:61-113.  Returns [dW, dFeat, dKernelPts, dPts, dSamples]."""
    pts, samples, neigh, kernel_pts = _f32(pts), _f32(samples), _i32(neigh), _f32(kernel_pts)
    basis, diff, npdf = kpconvn_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma)
    dw, dproj = _dense_grads(feat_basis_proj(basis, feats, neigh, ends), weights, in_grads)
    dfeat, dbasis = feat_basis_proj_grads(basis, feats, neigh, ends, dproj)
    aux = (dbasis / npdf).astype(np.float32)                                  # :103
    ddiff, dkp = _kp_basis_grads(diff, kernel_pts, sigma, aux)
    dpts, dsamples = _pt_diff_grads(pts.shape[0], samples.shape[0], neigh, radii, ddiff)
    return [dw, dfeat, dkp, dpts, dsamples]


def kpconvn_weight_var(pts, pdf, feats, samples, neigh, ends, radii, kernel_pts, sigma):
    """pccnn_lib_ops/pcconvs/kpconvn.cu:116-139."""
    basis, _, _ = kpconvn_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma)
    return variance_weights(basis, feats, neigh, ends)[0]


def gauss_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma):
    """kernel_pts_basis.cu:72-87 (fp32) then pccnn.cu:36-38: exp(-|kp - d|^2 / (2 sigma^2)) / pdf[n]."""
    pts, samples, neigh, kernel_pts = _f32(pts), _f32(samples), _i32(neigh), _f32(kernel_pts)
    _, diff = conv_basis(KP, pts, samples, neigh, radii, kernel_pts, sigma=1.0)
    diff_kp = kernel_pts[None, :, :] - diff[:, None, :]
    sq = diff_kp * diff_kp
    d2 = sq[..., 0]
    for i in range(1, sq.shape[-1]):
        d2 = d2 + sq[..., i]
    sig = np.float32(sigma)
    gauss = np.exp(-(d2 / (np.float32(2.0) * sig * sig))).astype(np.float32)
    npdf = _f32(pdf)[neigh[:, 0]].reshape(-1, 1)
    return (gauss / npdf).astype(np.float32), gauss, diff, diff_kp, npdf


def pccnn(pts, feats, pdf, samples, neigh, ends, radii, kernel_pts, sigma, weights):
    """pccnn_lib_ops/pcconvs/pccnn.cu:18-47."""
    basis = gauss_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma)[0]
    return _dense(feat_basis_proj(basis, feats, neigh, ends), weights)


def pccnn_grads(pts, feats, pdf, samples, neigh, ends, radii, kernel_pts, sigma, weights, in_grads):
    """pccnn_lib_ops/pcconvs/pccnn.cu:50-105 with kernel_pts_basis.cu:89-111.
    Returns [dW, dFeat, dKernelPts, dPdf, dPts, dSamples]."""
    pts, samples, neigh = _f32(pts), _f32(samples), _i32(neigh)
    basis, gauss, diff, diff_kp, npdf = gauss_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma)
    dw, dproj = _dense_grads(feat_basis_proj(basis, feats, neigh, ends), weights, in_grads)
    dfeat, dbasis = feat_basis_proj_grads(basis, feats, neigh, ends, dproj)
    npdf64, db64 = npdf.astype(np.float64), dbasis.astype(np.float64)
    dpdf_pair = ((-1.0 * basis.astype(np.float64) * db64) / npdf64).sum(axis=1)          # :91-92
    dpdf = np.zeros(_f32(pdf).shape[0], np.float64)
    np.add.at(dpdf, neigh[:, 0], dpdf_pair)
    gin = db64 / npdf64                                                                  # :98
    sig = np.float64(np.float32(sigma))
    gkp = -gin[..., None] * gauss.astype(np.float64)[..., None] * diff_kp.astype(np.float64) * (1.0 / (sig * sig))
    ddiff = (-gkp).sum(axis=1)
    dkp = gkp.sum(axis=0).astype(np.float32)
    dpts, dsamples = _pt_diff_grads(pts.shape[0], samples.shape[0], neigh, radii, ddiff)
    return [dw, dfeat, dkp, dpdf.astype(np.float32), dpts, dsamples]


def pccnn_weight_var(pts, feats, pdf, samples, neigh, ends, radii, kernel_pts, sigma):
    """pccnn_lib_ops/pcconvs/pccnn.cu:108-131."""
    basis = gauss_basis(pts, pdf, samples, neigh, radii, kernel_pts, sigma)[0]
    return variance_weights(basis, feats, neigh, ends)[0]


def pointconv_basis(pts, radii, samples, neigh, axis, bias):
    """pccnn_lib_ops/pcconvs/pointconv.cu:17-32: matmul(pt_diff, axis) + bias -> [T,K] (float64 sums, rounded)."""
    axis = _f32(axis)
    _, diff = conv_basis(KP, pts, samples, neigh, radii, np.zeros((1, 3), np.float32), sigma=1.0)
    out = diff.astype(np.float64) @ axis.astype(np.float64) + _f32(bias).reshape(1, -1).astype(np.float64)
    return out.astype(np.float32), diff


def pointconv_basis_grads(pts, radii, samples, neigh, axis, bias, in_grads):
    """pccnn_lib_ops/pcconvs/pointconv.cu:34-59.  Returns [dPts, dSamples, dAxis, dBias [1,K]]."""
    pts, samples, neigh, axis = _f32(pts), _f32(samples), _i32(neigh), _f32(axis)
    g = _f32(in_grads).astype(np.float64)
    _, diff = pointconv_basis(pts, radii, samples, neigh, axis, bias)
    dbias = g.sum(axis=0, keepdims=True).astype(np.float32)
    daxis = (diff.astype(np.float64).T @ g).astype(np.float32)
    ddiff = g @ axis.astype(np.float64).T
    dpts, dsamples = _pt_diff_grads(pts.shape[0], samples.shape[0], neigh, radii, ddiff)
    return [dpts, dsamples, daxis, dbias]


def pointconv(basis, feats, neigh, ends, weights):
    """pccnn_lib_ops/pcconvs/pointconv.cu:61-74."""
    return _dense(feat_basis_proj(basis, feats, neigh, ends), weights)


def pointconv_grads(basis, feats, neigh, ends, weights, in_grads):
    """pccnn_lib_ops/pcconvs/pointconv.cu:76-101.  Returns [dW, dFeat, dBasis]."""
    dw, dproj = _dense_grads(feat_basis_proj(basis, feats, neigh, ends), weights, in_grads)
    dfeat, dbasis = feat_basis_proj_grads(basis, feats, neigh, ends, dproj)
    return [dw, dfeat, dbasis]


def pointconv_weight_var(basis, feats, neigh, ends):
    """pccnn_lib_ops/pcconvs/pointconv.cu:103-111."""
    return variance_weights(basis, feats, neigh, ends)[0]


def _first_bin(values, edges):
    """spherical_basis.cu:42-46: first i with value <= edges[i], the last bin when there is none."""
    ids = np.full(values.shape[0], -1, np.int64)
    for i in range(edges.shape[0]):
        ids = np.where((values <= edges[i]) & (ids < 0), i, ids)
    return np.where(ids < 0, edges.shape[0] - 1, ids)


def spherical_basis(pts, samples, neigh, radii, radial_bins, azimuth_bins, polar_bins, with_angles=False):
    """spherical_basis.cu:24-66,136-156: one-hot [T, R*A*P+1]; fp32 distance, atan(y/(x+1e-6)),
    acos(clamp(z/(dist+1e-6), +-0.99999)); bin 0 holds pairs closer than 1e-4."""
    rb, ab, pb = _f32(radial_bins), _f32(azimuth_bins), _f32(polar_bins)
    _, diff = conv_basis(KP, pts, samples, neigh, radii, np.zeros((1, 3), np.float32), sigma=1.0)
    sq = diff * diff
    dist = np.sqrt((sq[:, 0] + sq[:, 1]) + sq[:, 2])
    azimuth = np.arctan(diff[:, 1] / (diff[:, 0] + np.float32(1e-6))).astype(np.float32)
    cosine = np.clip(diff[:, 2] / (dist + np.float32(1e-6)), np.float32(-0.99999), np.float32(0.99999))
    polar = np.arccos(cosine).astype(np.float32)
    ids = _first_bin(dist, rb) * (ab.shape[0] * pb.shape[0]) + _first_bin(azimuth, ab) * pb.shape[0] \
        + _first_bin(polar, pb) + 1
    ids = np.where(dist < 1e-4, 0, ids)
    k = rb.shape[0] * ab.shape[0] * pb.shape[0] + 1
    basis = np.zeros((diff.shape[0], k), np.float32)
    basis[np.arange(diff.shape[0]), ids] = 1.0
    if with_angles:
        return basis, (dist, azimuth, polar)
    return basis


def _counts(ends):
    ends = _i32(ends)
    return np.diff(np.concatenate([[0], ends])).astype(np.float32)


def sphconv(pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins, weights):
    """pccnn_lib_ops/pcconvs/sphconv.cu:18-51: correlation / (neighbor count + 1e-6)."""
    basis = spherical_basis(pts, samples, neigh, radii, radial_bins, azimuth_bins, polar_bins)
    out = _dense(feat_basis_proj(basis, feats, neigh, ends), weights)
    return (out / (_counts(ends).reshape(-1, 1) + np.float32(1e-6))).astype(np.float32)


def sphconv_grads(pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins, weights, in_grads):
    """pccnn_lib_ops/pcconvs/sphconv.cu:53-95.  Returns [dW, dFeat]."""
    basis = spherical_basis(pts, samples, neigh, radii, radial_bins, azimuth_bins, polar_bins)
    g = (_f32(in_grads) / (_counts(ends).reshape(-1, 1) + np.float32(1e-6))).astype(np.float32)
    dw, dproj = _dense_grads(feat_basis_proj(basis, feats, neigh, ends), weights, g)
    dfeat, _ = feat_basis_proj_grads(basis, feats, neigh, ends, dproj)
    return [dw, dfeat]


def sphconv_weight_var(pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins):
    """pccnn_lib_ops/pcconvs/sphconv.cu:97-117 with compute_variance_weights.cu:31-36 (pDivideNumNeighs = true):
    each sample's sum is scaled by 1 / count^2 before the mean."""
    basis = spherical_basis(pts, samples, neigh, radii, radial_bins, azimuth_bins, polar_bins)
    _, per = variance_weights(basis, feats, neigh, ends)
    cnt = _counts(ends).astype(np.float64)
    per = np.where(cnt > 0, per / np.maximum(cnt, 1.0) ** 2, 0.0)
    return np.float32(1.0 / per.mean())
