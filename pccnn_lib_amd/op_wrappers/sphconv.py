import torch

from .. import pccnn_lib_ops
from ._forward_only import ConvFunction, keeps_projection


class ComputeSPHConv(ConvFunction):
    """apply(pts, features, samples, neighbors, start_ids, radii, radial_bins, azimuz_bins, polar_bins, conv_weights)
    -> [M, Cout]: one-hot spherical-bin correlation divided by the neighbor count.  Only the features and the
    weights get gradients (pccnn_lib/op_wrappers/compute_sphconv.py:5-66)."""

    @staticmethod
    def forward(ctx, p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_radial_bins, p_azimuz_bins,
                p_polar_bins, p_conv_weights):
        keep = keeps_projection(ctx)          # no backward pass can follow: nothing is kept
        out = pccnn_lib_ops.sph_conv(p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                     p_radial_bins, p_azimuz_bins, p_polar_bins, p_conv_weights,
                                     return_proj=keep)
        out, proj = out if keep else (out, None)
        ctx.save_for_backward(p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_radial_bins,
                              p_azimuz_bins, p_polar_bins, p_conv_weights, proj)
        return out

    @staticmethod
    def backward(ctx, p_grads):
        pts, features, samples, neighbors, start_ids, radii, radial_bins, azimuz_bins, polar_bins, conv_weights, \
            proj = ctx.saved_tensors
        need = ctx.needs_input_grad
        ops = pccnn_lib_ops
        mask = (ops.GRAD_FEATS if need[1] else 0) | (ops.GRAD_WEIGHTS if need[9] else 0)
        mask |= pccnn_lib_ops.deterministic_flag()
        weight_grads, feat_grads = ops.sph_conv_grads(
            pts, features, samples, neighbors, start_ids, radii, radial_bins, azimuz_bins, polar_bins, conv_weights,
            p_grads, proj=proj, grad_mask=mask)
        return None, feat_grads, None, None, None, None, None, None, None, weight_grads


class ComputeSPHConvWeightVar(torch.autograd.Function):
    """apply(pts, features, samples, neighbors, start_ids, radii, radial_bins, azimuz_bins, polar_bins)
    (pccnn_lib/op_wrappers/compute_sphconv.py:69-107)."""

    @staticmethod
    def forward(ctx, p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii, p_radial_bins, p_azimuz_bins,
                p_polar_bins):
        return pccnn_lib_ops.sph_conv_weight_var(p_pts, p_features, p_samples, p_neighbors, p_start_ids, p_radii,
                                                 p_radial_bins, p_azimuz_bins, p_polar_bins)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None, None, None, None, None, None
