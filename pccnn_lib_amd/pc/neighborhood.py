import torch

from .. import pccnn_lib_ops


# A neighborhood over a grid that is not built yet (three dimensions, grid size known on the host) builds the grid and
# searches it in one native call (False: grid first, then the search, step by step; the result is the same).
ONE_CALL = True


class Neighborhood(object):
    """Radius neighborhood of the samples in a gridded cloud (pccnn_lib/pc/Neighborhood.py:10-53).

    ``neighbors_`` int32 [T, 2] = (original point index, sample index), grouped by ascending sample;
    ``start_ids_`` int32 [M] = inclusive running totals (the END of each sample's segment).
    The search radius is the grid's cell size (Neighborhood.py:44).  The sorted-index -> original-index
    remap of the reference (:47-53) happens inside the native fill pass."""

    def __init__(self, p_grid, p_samples, p_max_neighbors=0, p_key_order=False):
        """``p_key_order`` (not in the reference): keep the pair list with column 0 = index into the grid's sorted
        copy of the cloud, and make ``neighbors_`` from it only if somebody asks.  For a consumer that can work on
        the sorted copy (``layers.conv_base.point_side``)."""
        self.grid_ = p_grid
        self.samples_ = p_samples
        self.max_neighbors_ = p_max_neighbors
        self.mirror_ = False            # not computed yet; None = the neighborhood is not symmetric
        self.neighbors_key_order_ = None
        self.neighbors_original_ = None
        grid = p_grid
        with torch.no_grad():
            sample_pts = p_samples.pts_.detach()
            cloud = grid.pointcloud_
            if ONE_CALL and grid.cell_ids_ is None and grid.num_cells_device_ is None and cloud.pts_.shape[1] == 3 \
                    and sample_pts.shape[1] == 3 and cloud.pts_.shape[0] > 0 and sample_pts.shape[0] > 0 \
                    and grid.sized_on_host():
                # a grid that is not built yet, in three dimensions, sized from host values: grid, sample order,
                # count pass and pair total in one native call
                own = p_samples is cloud
                key_order = bool(p_key_order)
                built, neighbors, self.start_ids_ = pccnn_lib_ops.neighborhood_build(
                    cloud.pts_.detach(), cloud.batch_ids_, grid.bounding_box_.min_, grid.num_cells_host,
                    grid.cell_size_, cloud.batch_size_host(), None if own else sample_pts,
                    None if own else p_samples.batch_ids_, p_max_neighbors, not key_order)
                grid.adopt(built)
                if key_order:
                    self.neighbors_key_order_ = neighbors
                else:
                    self.neighbors_original_ = neighbors
                return
            if grid.cell_ids_ is None:
                grid.compute_cell_ids()
            grid.build_ds()
            # the samples go to the search in key order (a wavefront's 64 samples then share their cell walk and
            # read their coordinates as one run): the gridded cloud itself is sorted already
            if p_samples is grid.pointcloud_:
                sorted_keys, order, sorted_pts = grid.sorted_cell_ids_, grid.sorted_ids_i32_, grid.sorted_pts_
            else:
                sample_keys = pccnn_lib_ops.compute_keys(sample_pts, p_samples.batch_ids_, grid.bounding_box_.min_,
                                                         grid.num_cells_, grid.cell_size_)
                sorted_keys, order, sorted_pts = pccnn_lib_ops.sort_keys(sample_keys, grid.key_bits(), sample_pts)
            key_order = bool(p_key_order) and grid.sorted_pts_.shape[1] == 3
            neighbors, self.start_ids_ = pccnn_lib_ops.find_neighbors_ex(
                grid.sorted_pts_, grid.sorted_cell_ids_, sorted_pts, sorted_keys, grid.grid_ds_, grid.num_cells_,
                grid.cell_size_, p_max_neighbors, sample_order=order,
                point_remap=None if key_order else grid.sorted_ids_i32_, cell_table=grid.cell_table_,
                samples_presorted=True)
            if key_order:
                self.neighbors_key_order_ = neighbors
            else:
                self.neighbors_original_ = neighbors

    @property
    def neighbors_(self):
        """int32 [T, 2] (original point index, sample index) as in the reference."""
        if self.neighbors_original_ is None:
            with torch.no_grad():
                pairs = self.neighbors_key_order_
                point = torch.index_select(self.grid_.sorted_ids_i32_, 0, pairs[:, 0].to(torch.int64))
                self.neighbors_original_ = torch.stack((point, pairs[:, 1]), dim=1)
        return self.neighbors_original_

    @neighbors_.setter
    def neighbors_(self, p_value):
        self.neighbors_original_ = p_value
        self.neighbors_key_order_ = None

    def mirror(self):
        """int32 [T]: for every pair (a, b) the index of pair (b, a), when the samples are the gridded cloud
        itself and the search was not capped (then the pair list is symmetric); else None.  Computed on first
        use; the convolutions' backward passes use it to sum point gradients without atomics."""
        if self.mirror_ is False:
            self.mirror_ = None
            if self.samples_ is self.grid_.pointcloud_ and self.max_neighbors_ == 0:
                self.mirror_ = pccnn_lib_ops.mirror_pairs(self.neighbors_, self.start_ids_)
        return self.mirror_

    def __repr__(self):
        return "### Neighbors:\n{}\n### Start indices:\n{}".format(self.neighbors_, self.start_ids_)
