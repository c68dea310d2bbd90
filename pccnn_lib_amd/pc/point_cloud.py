import weakref

import numpy as np
import torch

from .. import pccnn_lib_ops
from ..op_wrappers import ComputePDF
from ._consts import device_vector, host_num_cells, host_vector


# compute_pdf without gradients (three dimensions, bandwidth known on the host) builds its grid and sums over it in
# one native call (False: Grid first, then the sum; the result is the same).
ONE_CALL = True


class Pointcloud(object):
    """A batch of point clouds stored flat (pccnn_lib/pc/Pointcloud.py:14-50): ``pts_`` float32 [N, D],
    ``batch_ids_`` int32 [N], ``batch_size_`` (0-d tensor), ``dim_manifold_``, and after ``compute_pdf``
    ``pts_unnorm_pdf_`` / ``pts_pdf_``."""

    def __init__(self, p_pts, p_batch_ids, p_manifold_dims=None, **kwargs):
        self.dim_manifold_ = p_pts.shape[1] if p_manifold_dims is None else p_manifold_dims
        self.pts_with_grads_ = False
        if 'requires_grad' in kwargs:
            self.pts_with_grads_ = kwargs['requires_grad']
            del kwargs['requires_grad']
        self.pts_ = torch.as_tensor(p_pts, **kwargs)
        self.batch_ids_ = torch.as_tensor(p_batch_ids, **kwargs)
        # batch ids that PointPooling selected carry the number of clouds along (a Poisson-disk selection keeps at
        # least one point of every cloud), which saves the read-back of their maximum
        self.batch_size_host_ = getattr(p_batch_ids, "pccnn_batch_size_", None)
        if self.batch_size_host_ is not None and (self.batch_ids_ is not p_batch_ids or p_batch_ids._version != 0):
            self.batch_size_host_ = None        # converted, moved or written to since the pooling made it
        self.batch_size_tensor_ = None
        if self.batch_size_host_ is None:
            self.batch_size_tensor_ = torch.max(self.batch_ids_) + 1
        # coordinates and batch ids that one PointPooling selected carry the box of the selection along (it came back
        # with the selection's size): the cloud starts with its bounding box known, as BoundingBox remembers it
        pooled = getattr(p_pts, "pccnn_pooled_box_", None)
        if pooled is not None and pooled is getattr(p_batch_ids, "pccnn_pooled_box_", None) \
                and self.pts_ is p_pts and self.batch_ids_ is p_batch_ids and p_pts._version == 0 \
                and p_batch_ids._version == 0:
            mn, mx, host = pooled.box
            self.aabb_cache_ = (weakref.ref(self.pts_), 0, weakref.ref(self.batch_ids_), 0, mn, mx, [host])
        self.num_pts_per_batch_ = None          # cached result of get_num_points_per_batch()
        if self.pts_with_grads_:
            self.pts_.requires_grad = True
        self.pts_pdf_ = None
        self.pts_unnorm_pdf_ = None

    @property
    def batch_size_(self):
        """0-d tensor max(batch_ids_) + 1 as in the reference (Pointcloud.py:38); made on first use when the number of
        clouds was already known on the host."""
        if self.batch_size_tensor_ is None:
            self.batch_size_tensor_ = torch.max(self.batch_ids_) + 1
        return self.batch_size_tensor_

    @batch_size_.setter
    def batch_size_(self, value):
        self.batch_size_tensor_ = value

    def to_device(self, p_device):
        self.pts_ = self.pts_.to(p_device)
        self.batch_ids_ = self.batch_ids_.to(p_device)
        if self.batch_size_tensor_ is not None:
            self.batch_size_tensor_ = self.batch_size_tensor_.to(p_device)
        if self.pts_unnorm_pdf_ is not None:
            self.pts_unnorm_pdf_ = self.pts_unnorm_pdf_.to(p_device)
            self.pts_pdf_ = self.pts_pdf_.to(p_device)

    def batch_size_host(self):
        """``batch_size_`` as a Python int (one read-back per cloud; the batch ids of a cloud do not change)."""
        if self.batch_size_host_ is None:
            self.batch_size_host_ = int(self.batch_size_)
        return self.batch_size_host_

    def get_num_points_per_batch(self):
        if self.num_pts_per_batch_ is None or self.num_pts_per_batch_.device != self.batch_ids_.device:
            with torch.no_grad():
                self.num_pts_per_batch_ = torch.bincount(self.batch_ids_.to(torch.int64),
                                                         minlength=self.batch_size_host()).to(torch.int32)
        return self.num_pts_per_batch_

    def compute_pdf(self, p_badnwidth):
        """Kernel density estimate per point (Pointcloud.py:81-109): neighbors within 4 bandwidths, at most 300
        per point, Gaussian kernel; ``pts_pdf_`` is the estimate divided by the cloud's point count."""
        from .bounding_box import BoundingBox
        from .grid import Grid
        from .neighborhood import Neighborhood
        bandwidth = device_vector(p_badnwidth, self.pts_.shape[1], self.pts_.device)
        bandwidth_host = host_vector(bandwidth)
        # four bandwidths (exact in fp32: a power of two), from the host values when they are known
        radii = bandwidth * 4.0 if bandwidth_host is None else device_vector(bandwidth_host * np.float32(4.0),
                                                                             self.pts_.shape[1], self.pts_.device)
        radii_host = host_vector(radii)
        aabb = BoundingBox(self, radii_host is not None)
        if ONE_CALL and not self.pts_.requires_grad and self.pts_.shape[1] == 3 and radii_host is not None:
            # no gradient wanted, three dimensions, bandwidth known on the host: grid and sum in one native call
            with torch.no_grad():
                self.pts_unnorm_pdf_, self.pts_pdf_ = pccnn_lib_ops.pdf_cloud(
                    self.dim_manifold_, bandwidth, self.pts_.detach(), self.batch_ids_, aabb.min_, radii,
                    lambda: host_num_cells(aabb.host(), radii_host), self.batch_size_host(), 300)
            return
        grid = Grid(self, aabb, radii)
        grid.compute_cell_ids()
        grid.build_ds()
        if self.pts_.requires_grad:
            neigh = Neighborhood(grid, self, 300)
            self.pts_unnorm_pdf_ = ComputePDF.apply(self.pts_, neigh.neighbors_, neigh.start_ids_, bandwidth,
                                                    self.dim_manifold_)
        elif self.pts_.shape[1] == 3:
            # no gradient wanted, three dimensions: the sum straight from the grid, without a pair list
            with torch.no_grad():
                self.pts_unnorm_pdf_, self.pts_pdf_ = pccnn_lib_ops.compute_pdf_grid(
                    self.dim_manifold_, bandwidth, grid.sorted_pts_, grid.sorted_cell_ids_, grid.sorted_ids_i32_,
                    grid.grid_ds_, grid.num_cells_, grid.cell_size_, 300, cell_table=grid.cell_table_,
                    with_normalized=True)
            return
        else:
            # no gradient wanted: keep the pair list in sorted-index space (no remap) and gather the
            # neighbor coordinates from the sorted copy of the points, where they are contiguous
            with torch.no_grad():
                neigh_sorted, ends = pccnn_lib_ops.find_neighbors_ex(
                    grid.sorted_pts_, grid.sorted_cell_ids_, grid.sorted_pts_, grid.sorted_cell_ids_, grid.grid_ds_,
                    grid.num_cells_, grid.cell_size_, 300, sample_order=grid.sorted_ids_i32_,
                    cell_table=grid.cell_table_, samples_presorted=True)
                self.pts_unnorm_pdf_ = pccnn_lib_ops.compute_pdf_sorted(
                    self.dim_manifold_, bandwidth, grid.sorted_pts_, self.pts_, neigh_sorted, ends)
        num_pts = torch.index_select(self.get_num_points_per_batch(), 0, self.batch_ids_.to(torch.int64))
        self.pts_pdf_ = self.pts_unnorm_pdf_ / num_pts.to(torch.float32)

    def global_pooling(self, p_in_tensor, p_pooling_method="avg"):
        """Per-cloud reduction of a per-point tensor (Pointcloud.py:113-131)."""
        index = self.batch_ids_.to(torch.int64).reshape(-1, 1).expand(-1, p_in_tensor.shape[1])
        out = torch.zeros((self.batch_size_host(), p_in_tensor.shape[1]), dtype=p_in_tensor.dtype,
                          device=p_in_tensor.device)
        reduce = {"max": "amax", "min": "amin", "avg": "mean", "sum": "sum"}[p_pooling_method]
        return out.scatter_reduce(0, index, p_in_tensor, reduce=reduce, include_self=False)

    def global_upsample(self, p_in_tensor):
        return torch.index_select(p_in_tensor, 0, self.batch_ids_.to(torch.int64))

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        """torch functions take a Pointcloud where they take a tensor (pccnn_lib/pc/Pointcloud.py:158-165): the call
        runs on the coordinates, and its result comes back as a new Pointcloud with the batch ids of the first cloud
        among the arguments, so ``torch.add(cloud, offset)`` or ``torch.mul(cloud, 2.0)`` move or scale a batch."""
        first = next(a for a in args if isinstance(a, Pointcloud))
        plain = [a.pts_ if hasattr(a, "pts_") else a for a in args]
        return Pointcloud(func(*plain, **(kwargs or {})), first.batch_ids_)

    def __repr__(self):
        return "### Points:\n{}\n### Batch Ids:\n{}\n### Batch Size:\n{}\n### Pdf:\n{}".format(
            self.pts_, self.batch_ids_, self.batch_size_, self.pts_pdf_)
