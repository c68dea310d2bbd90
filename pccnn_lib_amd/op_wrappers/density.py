import torch

from .. import pccnn_lib_ops


class ComputePDF(torch.autograd.Function):
    """apply(pts, neighbors, start_ids, bandwidth, manifold_dims) -> unnormalised density per point.
    Argument order differs from the native op's on purpose (pccnn_lib/op_wrappers/compute_pdf.py:14-35);
    tensors are saved, and point gradients returned, only when pts requires grad (:25-28, :47-56)."""

    @staticmethod
    def forward(ctx, p_pts, p_neighbors, p_start_ids, p_bandwidth, p_manifold_dims):
        if p_pts.requires_grad:
            ctx.save_for_backward(p_pts, p_neighbors, p_start_ids, p_bandwidth)
            ctx.manifold_dims_ = p_manifold_dims
        return pccnn_lib_ops.compute_pdf(p_manifold_dims, p_bandwidth, p_pts, p_neighbors, p_start_ids)

    @staticmethod
    def backward(ctx, p_grads):
        point_grads = None
        if len(ctx.saved_tensors) > 0:
            pts, neighbors, start_ids, bandwidth = ctx.saved_tensors
            point_grads = pccnn_lib_ops.compute_pdf_grads(ctx.manifold_dims_, bandwidth, pts, neighbors, start_ids,
                                                          p_grads)
        return point_grads, None, None, None, None
