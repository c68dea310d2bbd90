import torch

from .. import pccnn_lib_ops as _ops


class ComputePDF(torch.autograd.Function):
    """apply(pts, neighbors, start_ids, bandwidth, manifold_dims) -> unnormalised density per point.
    Argument order differs from the native op's on purpose (pccnn_lib/op_wrappers/compute_pdf.py:14-35);
    tensors are saved, and point gradients returned, only when pts requires grad (:25-28, :47-56)."""

    ARITY = 5

    @staticmethod
    def forward(ctx, *inputs):
        cloud, pairs, offsets, widths, manifold = inputs
        ctx.wants_points_ = bool(cloud.requires_grad)
        if ctx.wants_points_:
            ctx.manifold_dims_ = manifold
            ctx.save_for_backward(cloud, pairs, offsets, widths)
        return _ops.compute_pdf(manifold, widths, cloud, pairs, offsets)

    @staticmethod
    def backward(ctx, upstream):
        answer = [None] * ComputePDF.ARITY
        if ctx.wants_points_:
            cloud, pairs, offsets, widths = ctx.saved_tensors
            answer[0] = _ops.compute_pdf_grads(ctx.manifold_dims_, widths, cloud, pairs, offsets, upstream)
        return tuple(answer)
