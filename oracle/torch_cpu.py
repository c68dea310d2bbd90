"""Vectorised fp32 form of the Monte-Carlo convolution training step in torch on the CPU, all cores.

Test infrastructure like the rest of this directory: it is the multi-threaded CPU baseline that bench.py times beside
the GPU path, and tests/ check it against the scalar oracle.  Nothing in the product imports it.

The formulation is the one the reference's own tests use to check the CUDA ops (pccnn_lib/py_utils unit tests,
test_mcconv.py:65-91: gather the neighbor's coordinates and features per pair, evaluate the hidden layer on every
pair at once, sum the outer products of features and hidden outputs over each sample's list, one matrix product with
the weights), with torch's autograd for the backward pass as in test_mcconv_grads.py:127-141.  Semantics of the op:
pccnn_lib_ops/pcconvs/mcconv.cu:32-143, mlp_basis.cu:27-96 (leaky slope 0.2, division by the neighbor's density),
feat_basis_proj.cu:32-75 (projection laid out [M, Cin, K]).
"""
import numpy as np
import torch


def mcconv_step(pts, pdf, feats, neigh, ends, radii, axis, bias, weights, out_grads, samples_per_chunk=4096):
    """Forward and all gradients of one MCConv layer whose samples are the points themselves.

    pts f32[N,D], pdf f32[N], feats f32[N,Cin], neigh i32[T,2] (point, sample) sorted by sample, ends i32[N]
    (inclusive), radii f32[D], axis f32[D,K], bias f32[1,K], weights f32[1,K*Cin,Cout], out_grads f32[N,Cout].
    Returns (out, {"weights", "feats", "axis", "bias", "pdf", "pts"}) as numpy arrays; the gradient of the points sums
    their two roles (neighbor and sample).  Per chunk of samples the ragged neighbor lists are padded to the longest one,
    so the projection is one batched matrix product ([Cin, width] x [width, K] per sample) instead of a scatter-add of
    per-pair outer products, which is several times faster on a CPU.
    """
    t_pts = torch.from_numpy(np.ascontiguousarray(pts, np.float32)).requires_grad_(True)
    t_pdf = torch.from_numpy(np.ascontiguousarray(pdf, np.float32)).requires_grad_(True)
    t_feats = torch.from_numpy(np.ascontiguousarray(feats, np.float32)).requires_grad_(True)
    t_axis = torch.from_numpy(np.ascontiguousarray(axis, np.float32)).requires_grad_(True)
    t_bias = torch.from_numpy(np.ascontiguousarray(bias, np.float32).reshape(1, -1)).requires_grad_(True)
    t_w = torch.from_numpy(np.ascontiguousarray(weights, np.float32)).requires_grad_(True)
    t_g = torch.from_numpy(np.ascontiguousarray(out_grads, np.float32))
    inv_r = torch.from_numpy(1.0 / np.asarray(radii, np.float32))
    nb = torch.from_numpy(np.ascontiguousarray(neigh, np.int64))
    ends64 = np.asarray(ends, np.int64)
    m = ends64.shape[0]
    c_in, k = t_feats.shape[1], t_axis.shape[1]
    assert t_w.shape[0] == 1 and t_w.shape[1] == k * c_in
    out = torch.empty((m, t_w.shape[2]), dtype=torch.float32)
    starts64 = np.concatenate([[0], ends64[:-1]])
    for s0 in range(0, m, samples_per_chunk):
        s1 = min(m, s0 + samples_per_chunk)
        # the ragged neighbor lists of the chunk as a [samples, longest list] table of pair indices, short lists
        # padded with their own first pair and masked out of the hidden layer's output
        first = torch.from_numpy(starts64[s0:s1])
        count = torch.from_numpy(ends64[s0:s1] - starts64[s0:s1])
        width = max(1, int(count.max())) if s1 > s0 else 1
        slot = torch.arange(width).unsqueeze(0)
        valid = slot < count.unsqueeze(1)                                        # [samples, width]
        pair = torch.where(valid, first.unsqueeze(1) + slot, first.unsqueeze(1)).clamp_(max=max(nb.shape[0] - 1, 0))
        pt_i = nb[:, 0][pair]                                                    # [samples, width]
        smp_i = torch.arange(s0, s1).unsqueeze(1).expand(-1, width)
        diff = (t_pts[pt_i] - t_pts[smp_i]) * inv_r                              # [samples, width, D]
        act = torch.nn.functional.leaky_relu(diff @ t_axis + t_bias, 0.2)
        basis = act / t_pdf[pt_i].unsqueeze(2) * valid.unsqueeze(2)              # [samples, width, K]
        proj = torch.bmm(t_feats[pt_i].transpose(1, 2), basis)                   # [samples, Cin, K]
        o = proj.reshape(s1 - s0, c_in * k) @ t_w[0]
        out[s0:s1] = o.detach()
        (o * t_g[s0:s1]).sum().backward()
    grads = {"weights": t_w.grad, "feats": t_feats.grad, "axis": t_axis.grad, "bias": t_bias.grad, "pdf": t_pdf.grad,
             "pts": t_pts.grad}
    return out.numpy(), {key: val.numpy() for key, val in grads.items()}


def kpconv_step(pts, feats, neigh, ends, radii, kernel_pts, sigma, weights, out_grads, samples_per_chunk=2048):
    """Forward and the gradients w.r.t. weights, features and point positions of one KPConv layer whose samples are the
    points themselves, in the padded batched form of mcconv_step.

    The formulation is the one of the reference's test (test_kpconv.py:60-82): offsets (p - s) / r per pair, linear
    correlation max(0, 1 - |kernel point - offset| / sigma) with every kernel point (kernel_pts_basis.cu:41-70), the
    projection [M, Cin, K], one product with the weights f32[K*Cin, Cout]; autograd for the backward pass.
    Returns (out, {"weights", "feats", "pts"}); the gradient of the points sums their two roles."""
    t_pts = torch.from_numpy(np.ascontiguousarray(pts, np.float32)).requires_grad_(True)
    t_feats = torch.from_numpy(np.ascontiguousarray(feats, np.float32)).requires_grad_(True)
    t_w = torch.from_numpy(np.ascontiguousarray(weights, np.float32)).requires_grad_(True)
    t_kp = torch.from_numpy(np.ascontiguousarray(kernel_pts, np.float32))
    t_g = torch.from_numpy(np.ascontiguousarray(out_grads, np.float32))
    inv_r = torch.from_numpy(1.0 / np.asarray(radii, np.float32))
    nb = torch.from_numpy(np.ascontiguousarray(neigh, np.int64))
    ends64 = np.asarray(ends, np.int64)
    m = ends64.shape[0]
    c_in, k = t_feats.shape[1], t_kp.shape[0]
    assert tuple(t_w.shape[:1]) == (k * c_in,)
    out = torch.empty((m, t_w.shape[1]), dtype=torch.float32)
    starts64 = np.concatenate([[0], ends64[:-1]])
    for s0 in range(0, m, samples_per_chunk):
        s1 = min(m, s0 + samples_per_chunk)
        first = torch.from_numpy(starts64[s0:s1])
        count = torch.from_numpy(ends64[s0:s1] - starts64[s0:s1])
        width = max(1, int(count.max())) if s1 > s0 else 1
        slot = torch.arange(width).unsqueeze(0)
        valid = slot < count.unsqueeze(1)
        pair = torch.where(valid, first.unsqueeze(1) + slot, first.unsqueeze(1)).clamp_(max=max(nb.shape[0] - 1, 0))
        pt_i = nb[:, 0][pair]
        smp_i = torch.arange(s0, s1).unsqueeze(1).expand(-1, width)
        diff = (t_pts[pt_i] - t_pts[smp_i]) * inv_r                              # [samples, width, D]
        # distance without torch.norm: its gradient at distance zero (a self pair on the centre kernel point) is
        # NaN, the op's is zero
        sq = ((t_kp.view(1, 1, k, -1) - diff.unsqueeze(2)) ** 2).sum(dim=3)
        dist = torch.where(sq > 0, torch.sqrt(torch.where(sq > 0, sq, torch.ones_like(sq))), torch.zeros_like(sq))
        basis = torch.clamp(1.0 - dist / float(sigma), min=0.0) * valid.unsqueeze(2)
        proj = torch.bmm(t_feats[pt_i].transpose(1, 2), basis)                   # [samples, Cin, K]
        o = proj.reshape(s1 - s0, c_in * k) @ t_w
        out[s0:s1] = o.detach()
        (o * t_g[s0:s1]).sum().backward()
    grads = {"weights": t_w.grad, "feats": t_feats.grad, "pts": t_pts.grad}
    return out.numpy(), {key: val.numpy() for key, val in grads.items()}
