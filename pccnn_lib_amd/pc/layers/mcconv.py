import math

import torch

from ...op_wrappers import ComputeMCConv, ComputeMCConvWeightVar
from .conv_base import IConvLayer, IConvLayerFactory, mirror_if_needed, point_side, density_times_volume


class MCConv(IConvLayer):
    """Monte-Carlo convolution with a one-hidden-layer kernel (pccnn_lib/pc/layers/MCConv.py:11-140).
    Parameters keep the reference's names and shapes: ``proj_axis_`` [D, H*m], ``proj_bias_`` [1, H*m],
    ``conv_weights_`` [m, H*Cin, Cout/m].  The input cloud must carry a density (``compute_pdf``); the op
    receives it multiplied by the product of the radii (MCConv.py:93-94).  ``contraction_`` ("f32" by default;
    "bf16" = bf16 operands with fp32 accumulation, a mode the reference does not have) selects the precision of the
    [M, H*Cin] x [H*Cin, Cout] products of the forward and backward pass."""

    key_order_capable_ = True

    def __init__(self, p_dims, p_in_features, p_out_features, p_hidden_size, p_num_mlps=1,
                 p_constant_weight_var=True, p_const_var_value=1.0):
        IConvLayer.__init__(self, p_dims, p_in_features, p_out_features, p_constant_weight_var, p_const_var_value)
        self.hidden_size_, self.num_mlps_, self.contraction_ = p_hidden_size, p_num_mlps, "f32"
        hidden_total = p_hidden_size * p_num_mlps
        self._new_parameters(proj_axis_=(p_dims, hidden_total), proj_bias_=(1, hidden_total),
                             conv_weights_=(p_num_mlps, p_hidden_size * p_in_features, p_out_features // p_num_mlps))
        self.reset_parameters()

    def reset_parameters(self):
        self.conv_weights_.data.normal_(0.0, math.sqrt(1.0 / (self.feat_input_size_ * self.hidden_size_)))
        self.proj_axis_.data.normal_(0.0, math.sqrt(1.0 / self.num_dims_))
        self.proj_bias_.data.fill_(0.0)

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        if p_pc_in.pts_unnorm_pdf_ is None:
            raise RuntimeError("MCConv: the input point cloud has no density; call compute_pdf(bandwidth) first")
        cur_pdf = density_times_volume(p_pc_in.pts_unnorm_pdf_, p_radius)
        if torch.is_grad_enabled() and cur_pdf.requires_grad:
            pts, pairs, pdf, feats = p_pc_in.pts_, p_neighborhood.neighbors_, cur_pdf, p_in_features
        else:
            pts, pairs, pdf, feats = point_side(p_pc_in, p_neighborhood, cur_pdf, p_in_features)
        geometry = (pts, pdf, feats, p_pc_out.pts_, pairs, p_neighborhood.start_ids_, p_radius, self.proj_axis_,
                    self.proj_bias_)
        self._warm_up(lambda: ComputeMCConvWeightVar.apply(*geometry) * self.num_mlps_)
        return ComputeMCConv.apply(*geometry, self.conv_weights_, mirror_if_needed(p_neighborhood, pts, pdf),
                                   self.contraction_)


class MCConvFactory(IConvLayerFactory):
    def __init__(self, p_num_basis, p_const_var_w_init=False, p_num_mlps=1, p_const_var_value=1.0):
        super(MCConvFactory, self).__init__(p_num_basis, p_const_var_w_init, p_const_var_value)
        self.num_mlps_ = p_num_mlps

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        return self._remember(MCConv(p_dims, p_in_features, p_out_features, self.num_basis_, self.num_mlps_,
                                     self.conv_var_w_init_, self.const_var_value_))
