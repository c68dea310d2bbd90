import math

import torch

from ...op_wrappers import ComputePointConvBasis, ComputePointConv, ComputePointConvWeightVar
from .conv_base import IConvLayer, IConvLayerFactory
from .norm import GroupNormalization


class PointConv(IConvLayer):
    """PointConv (pccnn_lib/pc/layers/PointConv.py:9-200): basis = relu(affine map of the offsets) scaled by a small
    network of the relative inverse density of each neighbor, then the correlation with explicit basis values.
    Parameters ``proj_axis_`` [D, H], ``proj_bias_`` [1, H], ``conv_weights_`` [H*Cin, Cout], sub-module
    ``pdf_mlp_`` (1 -> 16 -> 1, sigmoid) and the optional ``basis_bn_`` / ``basis_gn_`` keep the reference's names."""

    def __init__(self, p_dims, p_in_features, p_out_features, p_hidden_size, p_constant_weight_var=True,
                 p_const_var_value=1.0, p_use_bn=False, p_use_gn=False, p_gn_size=32):
        super(PointConv, self).__init__(p_dims, p_in_features, p_out_features, p_constant_weight_var,
                                        p_const_var_value)
        self.use_bn_, self.use_gn_, self.gn_size_ = p_use_bn, p_use_gn, p_gn_size
        self.hidden_size_, self.init_proj_axis_ = p_hidden_size, False
        self._new_parameters(proj_axis_=(p_dims, p_hidden_size), proj_bias_=(1, p_hidden_size),
                             conv_weights_=(p_hidden_size * p_in_features, p_out_features))
        self.pdf_mlp_ = self._density_network(16, p_use_bn or p_use_gn)
        if p_use_bn:
            self.basis_bn_ = torch.nn.BatchNorm1d(p_hidden_size)
        elif p_use_gn:
            self.basis_gn_ = GroupNormalization(p_hidden_size, p_gn_size)
        self.reset_parameters()

    @staticmethod
    def _density_network(p_width, p_normalised):
        """1 -> width -> 1 with a sigmoid at the end; a batch norm behind each linear map when the layer normalises
        its basis (module indices as in the reference, so its state dicts load)."""
        def block(n_in, n_out, activation):
            return [torch.nn.Linear(n_in, n_out)] + ([torch.nn.BatchNorm1d(n_out)] if p_normalised else []) + [activation]
        return torch.nn.Sequential(*(block(1, p_width, torch.nn.ReLU()) + block(p_width, 1, torch.nn.Sigmoid())))

    def reset_parameters(self):
        self.conv_weights_.data.normal_(0.0, math.sqrt(2.0 / (self.feat_input_size_ * self.hidden_size_)))
        self.proj_axis_.data.normal_(0.0, math.sqrt(1.0 / self.num_dims_))
        self.proj_bias_.data.fill_(0.0)

    def __density_scale__(self, p_pc_in, p_neighborhood):
        """Inverse density of each neighbor relative to the largest one of its sample, through ``pdf_mlp_``."""
        pt_ids = p_neighborhood.neighbors_[:, 0].to(torch.int64)
        sample_ids = p_neighborhood.neighbors_[:, 1].to(torch.int64)
        inv_pdf = torch.reciprocal(torch.index_select(p_pc_in.pts_unnorm_pdf_, 0, pt_ids))
        num_samples = p_neighborhood.start_ids_.shape[0]
        max_inv = torch.zeros(num_samples, dtype=inv_pdf.dtype, device=inv_pdf.device)
        max_inv = max_inv.scatter_reduce(0, sample_ids, inv_pdf, reduce="amax", include_self=False)
        return self.pdf_mlp_(torch.reshape(inv_pdf / max_inv[sample_ids], (-1, 1)))

    def __basis__(self, p_pc_in, p_pc_out, p_neighborhood, p_radius, p_warmup):
        cur_radius = torch.ones_like(p_radius)
        basis_proj = ComputePointConvBasis.apply(p_pc_in.pts_, p_pc_out.pts_, p_neighborhood.neighbors_, cur_radius,
                                                 self.proj_axis_, self.proj_bias_)
        if self.use_bn_:
            basis_proj = self.basis_bn_(basis_proj)
        elif self.use_gn_ and p_warmup:
            # the reference calls its group norm here and drops the result (PointConv.py:139-140)
            self.basis_gn_(basis_proj, p_pc_out)
        return torch.relu(basis_proj)

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        cur_pdf = self.__density_scale__(p_pc_in, p_neighborhood)
        axis_stdv = torch.sqrt(1.0 / (self.num_dims_ * p_radius[0] * p_radius[0]))
        pairs, offsets = p_neighborhood.neighbors_, p_neighborhood.start_ids_
        warming = self.wamup_state_ and self.use_const_variance_init_
        if warming or self.init_proj_axis_:
            # the axes are redrawn for the radius at hand on every warm-up pass, and once after init_variance asked
            self.proj_axis_.data.normal_(0.0, float(axis_stdv))
            self.init_proj_axis_ = self.init_proj_axis_ and warming
        basis_proj = self.__basis__(p_pc_in, p_pc_out, p_neighborhood, p_radius, warming) * cur_pdf
        self._warm_up(lambda: ComputePointConvWeightVar.apply(basis_proj, p_in_features, pairs, offsets))
        return ComputePointConv.apply(basis_proj, p_in_features, pairs, offsets, self.conv_weights_)


class PointConvFactory(IConvLayerFactory):
    def __init__(self, p_num_basis, p_const_var_w_init=False, p_const_var_value=1.0, p_use_bn=False, p_use_gn=False,
                 p_gn_size=32):
        self.use_gn_ = p_use_gn
        self.use_bn_ = p_use_bn and not p_use_gn
        self.gn_size_ = p_gn_size
        super(PointConvFactory, self).__init__(p_num_basis, p_const_var_w_init, p_const_var_value)

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        return self._remember(PointConv(p_dims, p_in_features, p_out_features, self.num_basis_, self.conv_var_w_init_,
                                        self.const_var_value_, self.use_bn_, self.use_gn_, self.gn_size_))
