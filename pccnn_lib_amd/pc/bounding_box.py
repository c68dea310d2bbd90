import weakref

import torch

from .. import pccnn_lib_ops


class BoundingBox(object):
    """Per-cloud axis-aligned box padded by 1e-6 (pccnn_lib/pc/BoundingBox.py:10-18):
    ``min_`` and ``max_`` are float32 [B, D].  One native reduction replaces torch_scatter.

    A hierarchy level asks for the box of the same cloud several times (one grid each for pooling, density and the
    convolution's neighborhood), so the result is remembered on the cloud for as long as its coordinate and batch
    tensors are the same objects and have not been written to (torch's version counters).  A write through
    ``pts_.data`` or ``.detach()`` does not move those counters: after such a write, drop the entry
    (``del cloud.aabb_cache_``) or build a new Pointcloud, else grids keep using the old box."""

    def __init__(self, p_point_cloud, p_with_host=False):
        """``p_with_host`` (not in the reference): queue a copy of the box to the host right behind its kernels, for
        a caller that is about to size a grid from it on the host (``host()`` then only waits for that copy, and what
        the caller does in between runs beside the device); otherwise ``host()`` reads the box back when asked."""
        pts, ids = p_point_cloud.pts_, p_point_cloud.batch_ids_
        cached = getattr(p_point_cloud, "aabb_cache_", None)
        if cached is not None and cached[0]() is pts and cached[1] == pts._version and cached[2]() is ids \
                and cached[3] == ids._version:
            self.min_, self.max_, self.host_ = cached[4], cached[5], cached[6]
            return
        fetch = None
        if p_with_host:
            # the copy to the host is queued behind the box kernels; host() waits for it
            self.min_, self.max_, fetch = pccnn_lib_ops.bounding_box_host_later(pts.detach(), ids,
                                                                                p_point_cloud.batch_size_host())
        else:
            self.min_, self.max_ = pccnn_lib_ops.bounding_box(pts.detach(), ids, p_point_cloud.batch_size_host())
        # [the box on the host, or None; how to get it when a copy is on its way]: read back at most once and shared
        # by every user of the cache entry
        self.host_ = [None, fetch]
        # weak references: the entry neither keeps replaced tensors alive nor matches a new tensor at a reused address
        p_point_cloud.aabb_cache_ = (weakref.ref(pts), pts._version, weakref.ref(ids), ids._version, self.min_,
                                     self.max_, self.host_)

    def host(self):
        """(min, max) as float32 numpy arrays [B, D]: read back once per box, however many grids are laid over it."""
        if self.host_[0] is None:
            fetch = self.host_[1] if len(self.host_) > 1 else None
            if fetch is not None:
                self.host_[0] = fetch()
                self.host_[1] = None
            else:
                both = torch.stack([self.min_, self.max_]).cpu().numpy()
                self.host_[0] = (both[0], both[1])
        return self.host_[0]

    def __repr__(self):
        return "### Min:\n{}\n### Max:\n{}".format(self.min_, self.max_)
