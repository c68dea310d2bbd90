import math

import numpy as np
import torch

from ...op_wrappers import ComputeSPHConv, ComputeSPHConvWeightVar
from .conv_base import IConvLayer, IConvLayerFactory


def _upper_edges(p_extent, p_count):
    return torch.from_numpy(np.array([(p_extent / float(p_count)) * (i + 1) for i in range(p_count)], np.float32))


class SPHConv(IConvLayer):
    """Convolution over one-hot spherical bins (pccnn_lib/pc/layers/SPHConv.py:9-143): buffers ``radial_bins_``,
    ``azimuz_bins_``, ``polar_bins_`` hold the upper edges of equal bins over [0, 1], [0, 2 pi] and [0, pi];
    parameter ``conv_weights_`` [(R*A*P + 1) * Cin, Cout] ~ N(0, 1/(Cin * (R*A*P + 1)))."""

    def __init__(self, p_dims, p_in_features, p_out_features, p_num_radial_bins=1, p_num_azimuz_bins=5,
                 p_num_polar_bins=3, p_constant_weight_var=True, p_const_var_value=1.0):
        super(SPHConv, self).__init__(p_dims, p_in_features, p_out_features, p_constant_weight_var,
                                      p_const_var_value)
        counts = {"radial": (1.0, p_num_radial_bins), "azimuz": (2.0 * math.pi, p_num_azimuz_bins),
                  "polar": (math.pi, p_num_polar_bins)}
        self.num_basis_ = 1
        for label, (extent, count) in counts.items():
            setattr(self, "num_%s_bins_" % label, count)
            self.register_buffer("%s_bins_" % label, _upper_edges(extent, count))
            self.num_basis_ *= count
        self.num_basis_ += 1                    # one more bin for the sample itself
        self.sigma_cpu_ = None
        self._new_parameters(conv_weights_=(self.num_basis_ * p_in_features, p_out_features))
        self.reset_parameters()

    def reset_parameters(self):
        self.conv_weights_.data.normal_(0.0, math.sqrt(1.0 / (self.feat_input_size_ * self.num_basis_)))

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        geometry = (p_pc_in.pts_, p_in_features, p_pc_out.pts_, p_neighborhood.neighbors_, p_neighborhood.start_ids_,
                    p_radius, self.radial_bins_, self.azimuz_bins_, self.polar_bins_)
        self._warm_up(lambda: ComputeSPHConvWeightVar.apply(*geometry))
        return ComputeSPHConv.apply(*geometry, self.conv_weights_)


class SPHConvFactory(IConvLayerFactory):
    def __init__(self, p_num_radial_bins, p_num_azimuz_bins, p_num_polar_bins, p_const_var_w_init=False,
                 p_const_var_value=1.0):
        self.radial_bins_, self.azimuz_bins_, self.polar_bins_ = p_num_radial_bins, p_num_azimuz_bins, p_num_polar_bins
        IConvLayerFactory.__init__(self, p_num_radial_bins * p_num_azimuz_bins * p_num_polar_bins + 1,
                                   p_const_var_w_init, p_const_var_value)

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        return self._remember(SPHConv(p_dims, p_in_features, p_out_features, self.radial_bins_, self.azimuz_bins_,
                                      self.polar_bins_, self.conv_var_w_init_, self.const_var_value_))
