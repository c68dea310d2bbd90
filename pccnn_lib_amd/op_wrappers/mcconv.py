import torch

from .. import pccnn_lib_ops
from ._forward_only import ConvFunction, keeps_projection


class ComputeMCConv(ConvFunction):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, proj_axis, proj_bias, conv_weights)
    -> [M, Cout].  Gradients are routed to (pts, pdf, features, samples, -, -, -, proj_axis, proj_bias,
    conv_weights) (pccnn_lib/op_wrappers/compute_mcconv.py:14-75).  The projection built by the forward pass is
    kept for the backward pass, and only the gradients autograd asks for are computed.  An optional last argument takes the
    mirror index of a symmetric neighborhood (pccnn_lib_ops.mirror_pairs), used to sum point gradients without atomics;
    one more optional argument names the operand precision of the contraction ("f32", or "bf16" with fp32
    accumulation)."""

    @staticmethod
    def forward(ctx, p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_proj_axis,
                p_proj_bias, p_conv_weights, p_mirror=None, p_contraction="f32"):
        keep = keeps_projection(ctx)          # no backward pass can follow: nothing is kept
        out = pccnn_lib_ops.mc_conv(p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                    p_proj_axis, p_proj_bias, p_conv_weights, return_proj=keep,
                                    contraction=p_contraction)
        out, proj = out if keep else (out, None)
        ctx.contraction_ = p_contraction
        ctx.save_for_backward(p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_proj_axis,
                              p_proj_bias, p_conv_weights, proj)
        ctx.mirror_ = p_mirror
        return out

    @staticmethod
    def backward(ctx, p_grads):
        pts, pdf, features, samples, neighbors, start_ids, radii, axis, bias, conv_weights, proj = ctx.saved_tensors
        need = ctx.needs_input_grad
        ops = pccnn_lib_ops
        mask = (ops.GRAD_PTS if (need[0] or need[3]) else 0) | (ops.GRAD_PDF if need[1] else 0) \
            | (ops.GRAD_FEATS if need[2] else 0) | (ops.GRAD_BASIS_PARAMS if (need[7] or need[8]) else 0) \
            | (ops.GRAD_WEIGHTS if need[9] else 0)
        mask |= pccnn_lib_ops.deterministic_flag()
        weight_grads, feat_grads, axis_grads, bias_grads, pdf_grads, pt_grads, sample_grads = \
            ops.mc_conv_grads(pts, pdf, features, samples, neighbors, start_ids, radii, axis, bias, conv_weights,
                              p_grads, proj=proj, grad_mask=mask, mirror=ctx.mirror_,
                              contraction=ctx.contraction_)
        return pt_grads if need[0] else None, pdf_grads, feat_grads, sample_grads if need[3] else None, None, None, \
            None, axis_grads if need[7] else None, bias_grads if need[8] else None, weight_grads, None, None


class ComputeMCConvWeightVar(torch.autograd.Function):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, proj_axis, proj_bias): the statistic behind
    the variance-aware initialisation (pccnn_lib/op_wrappers/compute_mcconv.py:78-117)."""

    @staticmethod
    def forward(ctx, p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_proj_axis,
                p_proj_bias):
        return pccnn_lib_ops.mc_conv_weight_var(p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids,
                                                p_radii, p_proj_axis, p_proj_bias)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None, None, None, None, None, None
