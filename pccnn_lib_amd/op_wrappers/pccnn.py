import torch

from .. import pccnn_lib_ops
from ._forward_only import ConvFunction, keeps_projection


class ComputePCCNN(ConvFunction):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma, conv_weights) -> [M, Cout]:
    gaussian kernel-point correlation divided by the density of each neighbor.  Gradients go to
    (pts, pdf, features, samples, -, -, -, kernel_pts, -, conv_weights)
    (pccnn_lib/op_wrappers/compute_pccnn.py:5-67; the op itself takes features before pdf)."""

    @staticmethod
    def forward(ctx, p_pts, p_pt_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts, p_sigma,
                p_conv_weights, p_mirror=None):
        keep = keeps_projection(ctx)          # no backward pass can follow: nothing is kept
        out = pccnn_lib_ops.pccnn(p_pts, p_features, p_pt_pdf, p_samples, p_neighbors, p_start_ids, p_radii,
                                  p_kernel_pts, p_sigma, p_conv_weights, return_proj=keep)
        out, proj = out if keep else (out, None)
        ctx.save_for_backward(p_pts, p_pt_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts,
                              p_conv_weights, proj)
        ctx.sigma_ = p_sigma
        ctx.mirror_ = p_mirror
        return out

    @staticmethod
    def backward(ctx, p_grads):
        pts, pt_pdf, features, samples, neighbors, start_ids, radii, kernel_pts, conv_weights, proj = ctx.saved_tensors
        need = ctx.needs_input_grad
        ops = pccnn_lib_ops
        mask = (ops.GRAD_PTS if (need[0] or need[3]) else 0) | (ops.GRAD_PDF if need[1] else 0) \
            | (ops.GRAD_FEATS if need[2] else 0) | (ops.GRAD_BASIS_PARAMS if need[7] else 0) \
            | (ops.GRAD_WEIGHTS if need[9] else 0)
        mask |= pccnn_lib_ops.deterministic_flag()
        weight_grads, feat_grads, kernel_pts_grads, pt_pdf_grads, pt_grads, sample_grads = ops.pccnn_grads(
            pts, features, pt_pdf, samples, neighbors, start_ids, radii, kernel_pts, ctx.sigma_, conv_weights, p_grads,
            proj=proj, grad_mask=mask, mirror=ctx.mirror_)
        return pt_grads if need[0] else None, pt_pdf_grads, feat_grads, sample_grads if need[3] else None, None, \
            None, None, kernel_pts_grads, None, weight_grads, None


class ComputePCCNNWeightVar(torch.autograd.Function):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma)
    (pccnn_lib/op_wrappers/compute_pccnn.py:70-107)."""

    @staticmethod
    def forward(ctx, p_pts, p_pt_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts, p_sigma):
        return pccnn_lib_ops.pccnn_weight_variance(p_pts, p_features, p_pt_pdf, p_samples, p_neighbors, p_start_ids,
                                                   p_radii, p_kernel_pts, p_sigma)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None, None, None, None, None, None
