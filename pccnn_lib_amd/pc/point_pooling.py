import torch

from .. import pccnn_lib_ops
from .bounding_box import BoundingBox
from .grid import Grid
from ._consts import device_vector, host_num_cells, host_vector


# Three-dimensional Poisson-disk pooling with a cell size known on the host runs as one native call (False: the
# same steps one by one through Grid, as for every other case; the result is the same).
ONE_CALL = True


class PooledBox(object):
    """What the pooled coordinates and the pooled batch ids of one Poisson-disk pooling carry along: the bounding
    box of the selected points (device tensors and host copy), which came back with the selection's size.  A
    Pointcloud built from exactly these two tensors starts with its box known."""
    __slots__ = ("box",)

    def __init__(self, p_box):
        self.box = p_box


class PointPooling(object):
    """Point-cloud pooling (pccnn_lib/pc/PointPooling.py:16-102).

    ``poisson_disk``: a maximal subset of points no two of which are neighbors at the pooling radius, selected
    greedily in cell order; ``pooling_ids_`` holds the selected ORIGINAL point indices (int64).
    ``cell_average``: points are grouped by grid cell; ``pooling_ids_`` maps a point to its group."""

    # The one-call route queues its work and leaves the wait for the selection's size to the first use of one of
    # these four (LATER = False: waits in the constructor).  Whatever the caller queues in between - the cloud's
    # density, typically - runs on the device while the host waits for the count.
    LATER = True
    pooling_ids_ = property(lambda self: self._settled("ids"), lambda self, v: self._store("ids", v))
    pooled_box_ = property(lambda self: self._settled("box"), lambda self, v: self._store("box", v))
    pooled_pts_ = property(lambda self: self._settled("pts"), lambda self, v: self._store("pts", v))
    pooled_batch_ids_ = property(lambda self: self._settled("batch_ids"),
                                 lambda self, v: self._store("batch_ids", v))

    def _store(self, p_name, p_value):
        self.values_[p_name] = p_value

    def _settled(self, p_name):
        if self.pending_ is not None:
            finish, self.pending_ = self.pending_, None
            ids, box, pts, batch_ids = finish()
            self.values_.update(ids=ids, box=PooledBox(box) if box is not None else None, pts=pts,
                                batch_ids=batch_ids)
        return self.values_.get(p_name)

    def __del__(self):
        # a pooling nobody asked for: its queued copy to pinned memory has to land before that memory is released
        pending = getattr(self, "pending_", None)
        if pending is not None:
            try:
                pending.wait()
            except Exception:       # interpreter shutdown
                pass

    def __init__(self, p_point_cloud, p_radii, p_method="poisson_disk"):
        self.point_cloud_ = p_point_cloud
        self.radii_ = p_radii
        self.method_ = p_method
        self.pending_ = None
        self.values_ = {}
        self.pooled_box_ = None
        self.pooled_pts_ = self.pooled_batch_ids_ = None      # the cloud's own rows, when the pooling call gathered them
        with torch.no_grad():
            cell = device_vector(p_radii, p_point_cloud.pts_.shape[1], p_point_cloud.pts_.device)
            cell_host = host_vector(cell)
            bb = BoundingBox(p_point_cloud, cell_host is not None)
            if ONE_CALL and p_method == "poisson_disk" and p_point_cloud.pts_.shape[1] == 3:
                if cell_host is not None:
                    # three dimensions, cell size known on the host: grid, selection and its size in one native call
                    self.pending_ = pccnn_lib_ops.pool_poisson_later(
                        p_point_cloud.pts_.detach(), p_point_cloud.batch_ids_, bb.min_, cell,
                        lambda: host_num_cells(bb.host(), cell_host), p_point_cloud.batch_size_host())
                    if not self.LATER:
                        self._settled("ids")
                    return
            grid = Grid(p_point_cloud, bb, p_radii)
            grid.compute_cell_ids()
            if p_method == "poisson_disk":
                grid.build_ds()
                if grid.sorted_pts_.shape[1] == 3:
                    # three dimensions: the selection straight from the grid, same result as the two calls below
                    sampled = pccnn_lib_ops.poisson_disk_sampling_grid(
                        grid.sorted_pts_, grid.sorted_cell_ids_, grid.grid_ds_, grid.num_cells_, grid.cell_size_,
                        cell_table=grid.cell_table_).reshape(-1)
                else:
                    # self-neighborhood in sorted index space (PointPooling.py:58-62); the sorted points are
                    # already in key order, so the natural sample order is the cell order.
                    neighbors, start_ids = pccnn_lib_ops.find_neighbors_ex(
                        grid.sorted_pts_, grid.sorted_cell_ids_, grid.sorted_pts_, grid.sorted_cell_ids_,
                        grid.grid_ds_, grid.num_cells_, grid.cell_size_, 0, cell_table=grid.cell_table_)
                    sampled = pccnn_lib_ops.poisson_disk_sampling(grid.sorted_cell_ids_, neighbors, start_ids,
                                                                  grid.num_cells_).reshape(-1)
                self.pooling_ids_ = torch.index_select(grid.sorted_ids_, 0, sampled)
            elif p_method == "cell_average":
                unique_ids, inverse_ids = torch.unique(grid.cell_ids_, return_inverse=True)
                self.pooling_ids_ = inverse_ids
                self.num_pooling_pts_ = unique_ids.shape[0]
            else:
                raise RuntimeError("PointPooling: unknown method '%s'" % p_method)

    def pool_tensor(self, p_in_tensor, max_pool=False):
        if self.method_ == "poisson_disk":
            if p_in_tensor is self.point_cloud_.batch_ids_ and self.pooled_batch_ids_ is not None:
                out, self.pooled_batch_ids_ = self.pooled_batch_ids_, None          # handed out once
            elif p_in_tensor is self.point_cloud_.pts_ and self.pooled_pts_ is not None \
                    and not (torch.is_grad_enabled() and p_in_tensor.requires_grad):
                out, self.pooled_pts_ = self.pooled_pts_, None
            else:
                out = torch.index_select(p_in_tensor, 0, self.pooling_ids_)
            if p_in_tensor is self.point_cloud_.batch_ids_:
                # the selection keeps at least one point of every cloud: a Pointcloud built from these ids need not
                # read their maximum back
                out.pccnn_batch_size_ = self.point_cloud_.batch_size_host()
                out.pccnn_pooled_box_ = self.pooled_box_
            elif p_in_tensor is self.point_cloud_.pts_:
                out.pccnn_pooled_box_ = self.pooled_box_
            return out
        index = self.pooling_ids_.to(torch.int64).reshape(-1, 1).expand(-1, p_in_tensor.shape[1])
        out = torch.zeros((self.num_pooling_pts_, p_in_tensor.shape[1]), dtype=p_in_tensor.dtype,
                          device=p_in_tensor.device)
        return out.scatter_reduce(0, index, p_in_tensor, reduce="amax" if max_pool else "mean", include_self=False)
