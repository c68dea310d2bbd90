from .. import pccnn_lib_ops


class BoundingBox(object):
    """Per-cloud axis-aligned box padded by 1e-6 (pccnn_lib/pc/BoundingBox.py:10-18):
    ``min_`` and ``max_`` are float32 [B, D].  One native reduction replaces torch_scatter."""

    def __init__(self, p_point_cloud):
        self.min_, self.max_ = pccnn_lib_ops.bounding_box(
            p_point_cloud.pts_.detach(), p_point_cloud.batch_ids_, p_point_cloud.batch_size_host())

    def __repr__(self):
        return "### Min:\n{}\n### Max:\n{}".format(self.min_, self.max_)
