import math

import torch

from ... import pccnn_lib_ops
from .._consts import device_vector, host_vector


# A layer that can run on the grid's sorted copy of its input cloud (``point_side``) builds its own neighborhood in
# key order from this many input points on: a convolution over a large cloud whose points sit in memory in no
# spatial order gathers a cache line per pair and point (8 x 10^5 room points, 8 features, 8 M pairs: projection
# forward 255 -> 130 us, backward 506 -> 414 us).
KEY_ORDER_MIN_POINTS = 200000


def build_neighborhood(p_pc_in, p_pc_out, p_radius, p_max_neighs, p_key_order=False):
    """Box -> grid -> keys/sort -> pillar table -> neighbor search, as every layer of the reference does when no
    neighborhood is passed in (pccnn_lib/pc/layers/KPConv.py:142-146, MCConv.py:136-140)."""
    from ..bounding_box import BoundingBox
    from ..grid import Grid
    from ..neighborhood import Neighborhood
    radius = device_vector(p_radius, p_pc_in.pts_.shape[1], p_pc_in.pts_.device)
    bb = BoundingBox(p_pc_in, host_vector(radius) is not None)
    grid = Grid(p_pc_in, bb, radius)
    return Neighborhood(grid, p_pc_out, p_max_neighs, p_key_order)     # builds the grid


class _PermuteRows(torch.autograd.Function):
    """rows[perm]; the gradient goes back through the inverse permutation as a gather (no scatter-add)."""

    @staticmethod
    def forward(ctx, p_rows, p_perm, p_inverse):
        ctx.save_for_backward(p_inverse)
        return pccnn_lib_ops.gather_rows(p_rows.contiguous(), p_perm)

    @staticmethod
    def backward(ctx, p_grads):
        inverse, = ctx.saved_tensors
        return pccnn_lib_ops.gather_rows(p_grads.contiguous(), inverse), None, None


def point_side(p_pc_in, p_neighborhood, *p_per_point):
    """The point-side inputs of a convolution: (positions, pair list, per-point tensors...).

    Normally the cloud's own tensors and ``neighbors_``.  When the neighborhood kept its pairs in key order (a large
    cloud, see ``KEY_ORDER_MIN_POINTS``) and no gradient goes to the positions, the convolution runs
    on the grid's sorted copy of the cloud instead: positions from ``sorted_pts_``, the per-point tensors (features,
    densities) permuted once - with a gather in the backward pass too -, the pair list as it is.  Same pairs, same
    order inside a sample, same output; the kernels then read neighboring points from neighboring addresses."""
    nb = p_neighborhood
    pairs = getattr(nb, "neighbors_key_order_", None)
    if pairs is None or nb.grid_.pointcloud_ is not p_pc_in or \
            (torch.is_grad_enabled() and p_pc_in.pts_.requires_grad):
        return (p_pc_in.pts_, nb.neighbors_) + tuple(p_per_point)
    grid = nb.grid_
    perm, inverse = grid.sorted_ids_i32_, grid.inverse_sorted_ids()
    moved = []
    for x in p_per_point:
        if x is None:
            moved.append(None)
        elif torch.is_grad_enabled() and x.requires_grad:
            moved.append(_PermuteRows.apply(x, perm, inverse))
        else:
            moved.append(pccnn_lib_ops.gather_rows(x.detach().contiguous(), perm) if x.dtype == torch.float32
                         else torch.index_select(x, 0, perm.to(torch.int64)))
    return (grid.sorted_pts_, pairs) + tuple(moved)


def density_times_volume(p_pdf, p_radius):
    """``p_pdf * prod(p_radius)`` (pccnn_lib/pc/layers/MCConv.py:101-102).  For an isotropic radius given as a host
    value the product is taken on the host in fp32, (r * r) * r, which is what the device reduction of three equal
    numbers gives in any order, and multiplies the densities as a scalar: one launch instead of two."""
    import numpy as np
    host = host_vector(p_radius)
    if host is not None and host.size > 0 and bool(np.all(host == host[0])):
        prod = np.float32(1.0)
        for v in host:
            prod = np.float32(prod * v)
        return p_pdf * float(prod)
    return p_pdf * torch.prod(p_radius)


def mirror_if_needed(p_neighborhood, *p_geometry):
    """The neighborhood's mirror index when one of the tensors that receive point-side gradients (positions,
    densities) requires a gradient; None otherwise, or for a neighborhood object that has none."""
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in p_geometry) \
            and hasattr(p_neighborhood, "mirror"):
        return p_neighborhood.mirror()
    return None


class IConvLayer(torch.nn.Module):
    """Base of the point convolutions (pccnn_lib/pc/layers/IConvLayer.py:8-157):
    ``forward(pc_in, pc_out, in_features, radius, neighborhood=None, max_neighs=0)`` returns the output
    features, plus the neighborhood it built when none was given."""

    def __init__(self, p_dims, p_in_features, p_out_features, p_constant_weight_var=True, p_const_var_value=1.0):
        super(IConvLayer, self).__init__()
        self.num_dims_ = p_dims
        self.feat_input_size_ = p_in_features
        self.feat_output_size_ = p_out_features
        self.wamup_state_ = False
        self.use_const_variance_init_ = p_constant_weight_var
        self.out_constant_variance_ = p_const_var_value
        self.accum_weight_var_ = 0.0
        self.accum_weight_var_counter_ = 1.0

    def set_init_warmup_state(self, p_init_warmup_state):
        self.wamup_state_ = p_init_warmup_state

    def __update_weight_var__(self, p_new_var):
        self.accum_weight_var_ += (p_new_var - self.accum_weight_var_) / self.accum_weight_var_counter_
        self.accum_weight_var_counter_ += 1.0

    def _new_parameters(self, **p_shapes):
        """Register one uninitialised float32 parameter per keyword, in the order given (the order of the state dict
        and of ``parameters()``)."""
        for name, shape in p_shapes.items():
            setattr(self, name, torch.nn.Parameter(torch.empty(*shape)))

    def _warm_up(self, p_measure):
        """The variance-aware initialisation every layer shares (e.g. pccnn_lib/pc/layers/KPConv.py:103-116): in the
        warm-up state ``p_measure()`` returns this batch's weight-variance statistic, its reciprocal goes into the
        running mean, and the weights are redrawn with the variance that mean asks for.  Returns whether it ran."""
        if not (self.wamup_state_ and self.use_const_variance_init_):
            return False
        self.__update_weight_var__(1.0 / float(p_measure()))
        self.conv_weights_.data.normal_(0.0, math.sqrt(self.out_constant_variance_ / self.accum_weight_var_))
        return True

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        raise NotImplementedError

    key_order_capable_ = False          # the layer's __compute_convolution__ goes through point_side()

    def __create_neighborhood__(self, p_pc_in, p_pc_out, p_radius, p_max_neighs):
        key_order = self.key_order_capable_ and p_pc_in.pts_.shape[0] >= KEY_ORDER_MIN_POINTS and \
            not (torch.is_grad_enabled() and p_pc_in.pts_.requires_grad)
        return build_neighborhood(p_pc_in, p_pc_out, p_radius, p_max_neighs, key_order)

    def forward(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood=None, p_max_neighs=0):
        radius = device_vector(p_radius, self.num_dims_, p_pc_in.pts_.device)
        neighborhood = p_neighborhood
        if neighborhood is None:
            neighborhood = self.__create_neighborhood__(p_pc_in, p_pc_out, radius, p_max_neighs)
        out_features = self.__compute_convolution__(p_pc_in, p_pc_out, p_in_features, radius, neighborhood)
        if p_neighborhood is None:
            return out_features, neighborhood
        return out_features


class IConvLayerFactory(object):
    """Creates layers of one kind and remembers them (pccnn_lib/pc/layers/IConvLayer.py:160-215)."""

    def __init__(self, p_num_basis, p_const_var_w_init, p_const_var_value=1.0):
        self.num_basis_ = p_num_basis
        self.conv_var_w_init_ = p_const_var_w_init
        self.const_var_value_ = p_const_var_value
        self.conv_list_ = []

    def set_init_warmup_state_convs(self, p_state):
        for cur_conv in self.conv_list_:
            cur_conv.set_init_warmup_state(p_state)

    def define_num_basis(self, p_num_basis):
        self.num_basis_ = p_num_basis

    def _remember(self, p_layer):
        self.conv_list_.append(p_layer)
        return p_layer

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        raise NotImplementedError
