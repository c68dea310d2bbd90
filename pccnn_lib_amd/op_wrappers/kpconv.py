import torch

from .. import pccnn_lib_ops
from ._forward_only import ConvFunction, keeps_projection


class ComputeKPConv(ConvFunction):
    """apply(pts, features, samples, neighbors, start_ids, radii, kernel_pts, sigma, conv_weights) -> [M, Cout].
    Gradients are routed to (pts, features, samples, -, -, -, kernel_pts, -, conv_weights)
    (pccnn_lib/op_wrappers/compute_kpconv.py:14-73).  The projection built by the forward pass is kept for the
    backward pass, and only the gradients autograd asks for are computed.  An optional last argument takes the
    mirror index of a symmetric neighborhood (pccnn_lib_ops.mirror_pairs), used to sum point gradients without atomics;
    one more optional argument names the operand precision of the contraction ("f32", or "bf16" with fp32
    accumulation)."""

    @staticmethod
    def forward(ctx, p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts, p_sigma,
                p_conv_weights, p_mirror=None, p_contraction="f32"):
        keep = keeps_projection(ctx)          # no backward pass can follow: nothing is kept
        out = pccnn_lib_ops.kp_conv(p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                    p_kernel_pts, p_sigma, p_conv_weights, return_proj=keep,
                                    contraction=p_contraction)
        out, proj = out if keep else (out, None)
        ctx.contraction_ = p_contraction
        ctx.save_for_backward(p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts,
                              p_conv_weights, proj)
        ctx.sigma_ = p_sigma
        ctx.mirror_ = p_mirror
        return out

    @staticmethod
    def backward(ctx, p_grads):
        pts, features, samples, neighbors, start_ids, radii, kernel_pts, conv_weights, proj = ctx.saved_tensors
        need = ctx.needs_input_grad
        mask = (pccnn_lib_ops.GRAD_PTS if (need[0] or need[2]) else 0) | (pccnn_lib_ops.GRAD_FEATS if need[1] else 0) \
            | (pccnn_lib_ops.GRAD_BASIS_PARAMS if need[6] else 0) | (pccnn_lib_ops.GRAD_WEIGHTS if need[8] else 0)
        mask |= pccnn_lib_ops.deterministic_flag()
        weight_grads, feat_grads, kernel_pts_grads, pt_grads, sample_grads = pccnn_lib_ops.kp_conv_grads(
            pts, features, samples, neighbors, start_ids, radii, kernel_pts, ctx.sigma_, conv_weights, p_grads,
            proj=proj, grad_mask=mask, mirror=ctx.mirror_, contraction=ctx.contraction_)
        return pt_grads if need[0] else None, feat_grads, sample_grads if need[2] else None, None, None, None, \
            kernel_pts_grads, None, weight_grads, None, None


class ComputeKPConvWeightVar(torch.autograd.Function):
    """apply(pts, features, samples, neighbors, start_ids, radii, kernel_pts, sigma): the statistic behind the
    variance-aware initialisation (pccnn_lib/op_wrappers/compute_kpconv.py:76-113)."""

    @staticmethod
    def forward(ctx, p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_kernel_pts, p_sigma):
        return pccnn_lib_ops.kp_conv_weight_var(p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                                p_kernel_pts, p_sigma)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None, None, None, None, None
