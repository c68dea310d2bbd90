import torch

from .. import pccnn_lib_ops
from ._forward_only import ConvFunction, keeps_projection


class ComputeKPConvN(ConvFunction):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma, conv_weights) -> [M, Cout]:
    KPConv whose correlation is divided by the density of each neighbor.  Gradients go to
    (pts, -, features, samples, -, -, -, kernel_pts, -, conv_weights); the density gets none
    (pccnn_lib/op_wrappers/compute_kpconvn.py:9-74).  The projection of the forward pass is kept for the
    backward pass and only the gradients autograd asks for are computed.  An optional last argument takes the
    mirror index of a symmetric neighborhood (pccnn_lib_ops.mirror_pairs), used to sum point gradients without atomics."""

    @staticmethod
    def forward(ctx, p_pts, p_pdfs, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts, p_sigma,
                p_conv_weights, p_mirror=None):
        keep = keeps_projection(ctx)          # no backward pass can follow: nothing is kept
        out = pccnn_lib_ops.kp_conv_n(p_pts, p_pdfs, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                      p_kernel_pts, p_sigma, p_conv_weights, return_proj=keep)
        out, proj = out if keep else (out, None)
        ctx.save_for_backward(p_pts, p_pdfs, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts,
                              p_conv_weights, proj)
        ctx.sigma_ = p_sigma
        ctx.mirror_ = p_mirror
        return out

    @staticmethod
    def backward(ctx, p_grads):
        pts, pdfs, features, samples, neighbors, start_ids, radii, kernel_pts, conv_weights, proj = ctx.saved_tensors
        need = ctx.needs_input_grad
        ops = pccnn_lib_ops
        mask = (ops.GRAD_PTS if (need[0] or need[3]) else 0) | (ops.GRAD_FEATS if need[2] else 0) \
            | (ops.GRAD_BASIS_PARAMS if need[7] else 0) | (ops.GRAD_WEIGHTS if need[9] else 0)
        mask |= pccnn_lib_ops.deterministic_flag()
        weight_grads, feat_grads, kernel_pts_grads, pt_grads, sample_grads = ops.kp_conv_n_grads(
            pts, pdfs, features, samples, neighbors, start_ids, radii, kernel_pts, ctx.sigma_, conv_weights, p_grads,
            proj=proj, grad_mask=mask, mirror=ctx.mirror_)
        return pt_grads if need[0] else None, None, feat_grads, sample_grads if need[3] else None, None, None, \
            None, kernel_pts_grads, None, weight_grads, None


class ComputeKPConvNWeightVar(torch.autograd.Function):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma): the statistic behind the
    variance-aware initialisation (pccnn_lib/op_wrappers/compute_kpconvn.py:77-115)."""

    @staticmethod
    def forward(ctx, p_pts, p_pdfs, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts, p_sigma):
        return pccnn_lib_ops.kp_conv_n_weight_var(p_pts, p_pdfs, p_features, p_samples, p_neighbors, p_start_ids,
                                                  p_radii, p_kernel_pts, p_sigma)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None, None, None, None, None, None
