"""Index-producing ops: none of them propagates gradients (every backward returns None for each
input, as in pccnn_lib/op_wrappers/{compute_keys,build_grid_ds_funct,find_neighbors,poisson_disk_sampling}.py)."""
import torch

from .. import pccnn_lib_ops


class ComputeKeys(torch.autograd.Function):
    """apply(pts, batch_ids, aabb_min, grid_size, cell_size) -> int64 keys
    (pccnn_lib/op_wrappers/compute_keys.py:14-25)."""

    @staticmethod
    def forward(ctx, p_pts, p_batch_ids, p_aabb_min, p_grid_size, p_cell_size):
        return pccnn_lib_ops.compute_keys(p_pts, p_batch_ids, p_aabb_min, p_grid_size, p_cell_size)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None, None


class BuildGridDS(torch.autograd.Function):
    """apply(sorted_keys, grid_size, batch_size) -> int32 [B, nc0, nc1, 2]
    (pccnn_lib/op_wrappers/build_grid_ds_funct.py:10-23; batch_size is a 0-d tensor or an int)."""

    @staticmethod
    def forward(ctx, p_keys, p_grid_size, p_batch_size):
        batch = p_batch_size.tolist() if torch.is_tensor(p_batch_size) else int(p_batch_size)
        shape = [batch] + p_grid_size[0:2].tolist() + [2]
        return pccnn_lib_ops.build_grid_ds(p_keys, p_grid_size, shape)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None


class FindNeighbors(torch.autograd.Function):
    """apply(sorted_pts, sorted_keys, samples, sample_keys, grid_ds, grid_size, radius, max_neighbors)
    -> (neighbors int32 [T,2], start_ids int32 [M]) (pccnn_lib/op_wrappers/find_neighbors.py:14-31)."""

    @staticmethod
    def forward(ctx, p_pts, p_pt_keys, p_samples, p_sample_keys, p_grid_ds, p_grid_size, p_radius,
                p_max_neighbors):
        neigh, start_ids = pccnn_lib_ops.find_neighbors(
            p_pts, p_pt_keys, p_samples, p_sample_keys, p_grid_ds, p_grid_size, p_radius, p_max_neighbors)
        return neigh, start_ids

    @staticmethod
    def backward(ctx, p_grads_neigh, p_grads_start_ids):
        return None, None, None, None, None, None, None, None


class PoissonDiskSamlping(torch.autograd.Function):
    """apply(sorted_keys, neighbors, start_ids, grid_size) -> int64 [S,1] selected sorted indices
    (pccnn_lib/op_wrappers/poisson_disk_sampling.py:14-26; the class name keeps the reference's spelling)."""

    @staticmethod
    def forward(ctx, p_sorted_keys, p_neighbors, p_start_ids, p_grid_size):
        return pccnn_lib_ops.poisson_disk_sampling(p_sorted_keys, p_neighbors, p_start_ids, p_grid_size)

    @staticmethod
    def backward(ctx, p_grads):
        return None, None, None, None
