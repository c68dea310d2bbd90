import torch

from .. import pccnn_lib_ops
from ._forward_only import ConvFunction, keeps_projection


class ComputePointConvBasis(torch.autograd.Function):
    """apply(pts, samples, neighbors, radii, axis_proj, axis_bias) -> [T, K]: the affine map of the normalised
    offsets; gradients go to (pts, samples, -, -, axis_proj, axis_bias)
    (pccnn_lib/op_wrappers/compute_pointconv.py:5-58)."""

    @staticmethod
    def forward(ctx, p_pts, p_samples, p_neighbors, p_radii, p_axis_proj, p_axis_bias):
        ctx.save_for_backward(p_pts, p_samples, p_neighbors, p_radii, p_axis_proj, p_axis_bias)
        return pccnn_lib_ops.point_conv_basis(p_pts, p_radii, p_samples, p_neighbors, p_axis_proj, p_axis_bias)

    @staticmethod
    def backward(ctx, p_grads):
        pts, samples, neighbors, radii, axis_proj, axis_bias = ctx.saved_tensors
        pt_grads, sample_grads, axis_grad, bias_grad = pccnn_lib_ops.point_conv_basis_grads(
            pts, radii, samples, neighbors, axis_proj, axis_bias, p_grads)
        return pt_grads, sample_grads, None, None, axis_grad, bias_grad.reshape(axis_bias.shape)


class ComputePointConv(ConvFunction):
    """apply(basis_proj [T, K], features, neighbors, start_ids, conv_weights) -> [M, Cout]; gradients go to
    (basis_proj, features, -, -, conv_weights) (pccnn_lib/op_wrappers/compute_pointconv.py:61-107)."""

    @staticmethod
    def forward(ctx, p_basis_proj, p_features, p_neighbors, p_start_ids, p_conv_weights):
        p_basis_proj = p_basis_proj.contiguous()
        keep = keeps_projection(ctx)          # no backward pass can follow: nothing is kept
        out = pccnn_lib_ops.point_conv(p_basis_proj, p_features, p_neighbors, p_start_ids, p_conv_weights,
                                       return_proj=keep)
        out, proj = out if keep else (out, None)
        ctx.save_for_backward(p_basis_proj, p_features, p_neighbors, p_start_ids, p_conv_weights, proj)
        return out

    @staticmethod
    def backward(ctx, p_grads):
        basis_proj, features, neighbors, start_ids, conv_weights, proj = ctx.saved_tensors
        need = ctx.needs_input_grad
        ops = pccnn_lib_ops
        mask = (ops.GRAD_BASIS_PARAMS if need[0] else 0) | (ops.GRAD_FEATS if need[1] else 0) \
            | (ops.GRAD_WEIGHTS if need[4] else 0)
        mask |= pccnn_lib_ops.deterministic_flag()
        weights_grads, feat_grads, basis_grads = ops.point_conv_grads(
            basis_proj, features, neighbors, start_ids, conv_weights, p_grads, proj=proj, grad_mask=mask)
        return basis_grads, feat_grads, None, None, weights_grads


class ComputePointConvWeightVar(torch.autograd.Function):
    """apply(basis, features, neighbors, start_ids) (pccnn_lib/op_wrappers/compute_pointconv.py:110-139)."""

    @staticmethod
    def forward(ctx, p_basis, p_features, p_neighbors, p_start_ids):
        return pccnn_lib_ops.point_conv_weight_var(p_basis.contiguous(), p_features, p_neighbors, p_start_ids)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None
