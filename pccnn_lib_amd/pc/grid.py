import torch

from .. import pccnn_lib_ops
from ._consts import device_vector, host_num_cells, host_vector


class Grid(object):
    """Regular grid over a point cloud (pccnn_lib/pc/Grid.py:10-72).

    Attributes as in the reference: ``cell_size_``, ``num_cells_`` (int32 [D]), ``cell_ids_`` (int64 [N]),
    ``sorted_ids_`` (int64 [N]: the stable key-order permutation) and ``grid_ds_`` (int32 [B, nc0, nc1, 2]).
    The argsort and the gathers of sorted keys / points are one native radix sort; its by-products
    (``sorted_cell_ids_``, ``sorted_pts_``, ``sorted_ids_i32_``) are kept for Neighborhood and PointPooling, and
    for grids of up to 2^26 cells ``build_ds`` also builds ``cell_table_`` (first sorted index of every cell)."""

    def __init__(self, p_point_cloud, p_bounding_box, p_cell_size):
        self.pointcloud_ = p_point_cloud
        self.bounding_box_ = p_bounding_box
        self.cell_size_ = device_vector(p_cell_size, p_point_cloud.pts_.shape[1], p_point_cloud.pts_.device)
        self.num_cells_device_ = None
        self.num_cells_host_ = None
        self.cell_ids_ = None
        self.sorted_ids_i64_ = None
        self.sorted_ids_i32_ = None
        self.sorted_cell_ids_ = None
        self.sorted_pts_ = None
        self.grid_ds_ = None
        self.cell_table_ = None

    @property
    def num_cells_(self):
        """int32 [D] on the device (Grid.py:26-28: fp32 division, truncation, + 1, maximum over the clouds): computed
        there on first use, unless the grid was built from the host copy of the same numbers before."""
        if self.num_cells_device_ is None:
            with torch.no_grad():
                self.num_cells_device_ = pccnn_lib_ops.num_cells(self.bounding_box_.min_, self.bounding_box_.max_,
                                                                 self.cell_size_.contiguous())
        return self.num_cells_device_

    @num_cells_.setter
    def num_cells_(self, p_value):
        self.num_cells_device_ = p_value

    def sized_on_host(self):
        """True when the grid size can be had without a read-back of its own: the cell size came from host values
        and the box keeps a host copy."""
        return self.num_cells_host_ is not None or (host_vector(self.cell_size_) is not None
                                                    and hasattr(self.bounding_box_, "host"))

    def adopt(self, p_built):
        """Takes the tensors of ``pccnn_lib_ops.grid_build_sized`` as this grid's."""
        (self.num_cells_device_, self.cell_ids_, self.sorted_cell_ids_, self.sorted_ids_i32_, self.sorted_pts_,
         self.grid_ds_, self.cell_table_) = p_built

    @property
    def sorted_ids_(self):
        """int64 [N] permutation, as the reference keeps it; converted from the native int32 one on first use."""
        if self.sorted_ids_i64_ is None and self.sorted_ids_i32_ is not None:
            self.sorted_ids_i64_ = self.sorted_ids_i32_.to(torch.int64)
        return self.sorted_ids_i64_

    def inverse_sorted_ids(self):
        """int32 [N]: position of every point in the key order (the inverse of ``sorted_ids_``), made on first use."""
        if getattr(self, "inverse_sorted_ids_", None) is None:
            self.inverse_sorted_ids_ = pccnn_lib_ops.invert_permutation(self.sorted_ids_i32_)
        return self.inverse_sorted_ids_

    def num_cells_host(self):
        """``num_cells_`` as a list of ints.  When the cell size came from host values, the same fp32 arithmetic
        (subtract, IEEE divide, truncate, + 1, maximum over the clouds) runs in numpy on the box's host copy, which is
        read back once per cloud, not once per grid; otherwise the device result is read back."""
        if self.num_cells_host_ is None:
            cell = host_vector(self.cell_size_)
            if cell is not None and hasattr(self.bounding_box_, "host"):
                self.num_cells_host_ = host_num_cells(self.bounding_box_.host(), cell)
            else:
                self.num_cells_host_ = self.num_cells_.tolist()
        return self.num_cells_host_

    def key_bits(self):
        return pccnn_lib_ops.key_bits_for(self.num_cells_host(), self.pointcloud_.batch_size_host())

    def compute_cell_ids(self):
        """Keys and their stable order (Grid.py:40-53).  The native call that computes them also builds the pillar
        table (and the cell table of small grids), which ``build_ds`` then finds in place."""
        if self.cell_ids_ is None:
            with torch.no_grad():
                pts = self.pointcloud_.pts_.detach()
                batch = self.pointcloud_.batch_size_host()
                if self.num_cells_device_ is None and self.sized_on_host():
                    self.adopt(pccnn_lib_ops.grid_build_sized(pts, self.pointcloud_.batch_ids_, self.bounding_box_.min_,
                                                              self.num_cells_host(), self.cell_size_, batch))
                    return
                cells = self.num_cells_host()
                shape = [batch] + cells[0:2] + [2]
                total = batch
                for c in cells:
                    total *= c
                with_table = total if (len(cells) == 3 and total <= pccnn_lib_ops.CELL_TABLE_MAX_CELLS) else 0
                (self.cell_ids_, self.sorted_cell_ids_, self.sorted_ids_i32_, self.sorted_pts_, self.grid_ds_,
                 self.cell_table_) = pccnn_lib_ops.grid_build(pts, self.pointcloud_.batch_ids_,
                                                              self.bounding_box_.min_, self.num_cells_,
                                                              self.cell_size_, self.key_bits(), shape, with_table)

    def build_ds(self):
        if self.cell_ids_ is None or self.sorted_ids_i32_ is None:
            raise RuntimeError('In order to build the data structure first the keys for each point has to be '
                               'computed.')
        if self.grid_ds_ is None:
            with torch.no_grad():
                shape = [self.pointcloud_.batch_size_host()] + self.num_cells_host()[0:2] + [2]
                self.grid_ds_ = pccnn_lib_ops.build_grid_ds(self.sorted_cell_ids_, self.num_cells_, shape)
                cells = self.num_cells_host()
                total = self.pointcloud_.batch_size_host()
                for c in cells:
                    total *= c
                if len(cells) == 3 and total <= pccnn_lib_ops.CELL_TABLE_MAX_CELLS:
                    # per-cell start offsets: the search then needs no binary search inside a pillar
                    self.cell_table_ = pccnn_lib_ops.build_cell_table(self.sorted_cell_ids_, total)

    def __repr__(self):
        return "### Cell size:\n{}\n### Num cells:\n{}\n### Cell Ids:\n{}\n### Sorted Ids:\n{}\n### Grid Ds:\n{}".format(
            self.cell_size_, self.num_cells_, self.cell_ids_, self.sorted_ids_, self.grid_ds_)
