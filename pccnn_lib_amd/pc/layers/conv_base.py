import torch

from .._consts import device_vector


def build_neighborhood(p_pc_in, p_pc_out, p_radius, p_max_neighs):
    """Box -> grid -> keys/sort -> pillar table -> neighbor search, as every layer of the reference does when no
    neighborhood is passed in (pccnn_lib/pc/layers/KPConv.py:142-146, MCConv.py:136-140)."""
    from ..bounding_box import BoundingBox
    from ..grid import Grid
    from ..neighborhood import Neighborhood
    bb = BoundingBox(p_pc_in)
    grid = Grid(p_pc_in, bb, p_radius)
    grid.compute_cell_ids()
    grid.build_ds()
    return Neighborhood(grid, p_pc_out, p_max_neighs)


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

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        raise NotImplementedError

    def __create_neighborhood__(self, p_pc_in, p_pc_out, p_radius, p_max_neighs):
        return build_neighborhood(p_pc_in, p_pc_out, p_radius, p_max_neighs)

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

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        raise NotImplementedError
