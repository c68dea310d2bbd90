import torch

from .. import pccnn_lib_ops


class ComputeMCConv(torch.autograd.Function):
    """apply(pts, pdf, features, samples, neighbors, start_ids, radii, proj_axis, proj_bias, conv_weights)
    -> [M, Cout].  Gradients are routed to (pts, pdf, features, samples, -, -, -, proj_axis, proj_bias,
    conv_weights) (pccnn_lib/op_wrappers/compute_mcconv.py:14-75)."""

    @staticmethod
    def forward(ctx, p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_proj_axis,
                p_proj_bias, p_conv_weights):
        ctx.save_for_backward(p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_proj_axis,
                              p_proj_bias, p_conv_weights)
        return pccnn_lib_ops.mc_conv(p_pts, p_pdf, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                     p_proj_axis, p_proj_bias, p_conv_weights)

    @staticmethod
    def backward(ctx, p_grads):
        pts, pdf, features, samples, neighbors, start_ids, radii, axis, bias, conv_weights = ctx.saved_tensors
        weight_grads, feat_grads, axis_grads, bias_grads, pdf_grads, pt_grads, sample_grads = \
            pccnn_lib_ops.mc_conv_grads(pts, pdf, features, samples, neighbors, start_ids, radii, axis, bias,
                                        conv_weights, p_grads)
        return pt_grads, pdf_grads, feat_grads, sample_grads, None, None, None, axis_grads, bias_grads, weight_grads


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
