import math

import numpy as np
import torch

import time

from ...op_wrappers import ComputeKPConv, ComputeKPConvWeightVar, ComputeKPConvN, ComputeKPConvNWeightVar, \
    ComputePCCNN, ComputePCCNNWeightVar
from .conv_base import IConvLayer, IConvLayerFactory, mirror_if_needed, point_side, density_times_volume
from .kernel_points import kernel_pts_dict


def _seeded_rotation(seed):
    """Rotation about x, then y, then z by angles drawn from RandomState(seed), as
    pccnn_lib/py_utils/pc_utils.py:77-125 builds it (points are multiplied from the left: p @ R)."""
    ax, ay, az = (np.random.RandomState(seed).random_sample(3) - 0.5) * 2.0 * (2.0 * np.pi)
    rx = np.array([[1, 0, 0], [0, np.cos(ax), -np.sin(ax)], [0, np.sin(ax), np.cos(ax)]])
    ry = np.array([[np.cos(ay), 0, np.sin(ay)], [0, 1, 0], [-np.sin(ay), 0, np.cos(ay)]])
    rz = np.array([[np.cos(az), -np.sin(az), 0], [np.sin(az), np.cos(az), 0], [0, 0, 1]])
    return rz @ (ry @ rx)


def _kernel_point_buffers(p_dims, p_num_kernel_pts, p_sigma_scale, p_rotation_seed):
    """Layout normalised by its largest norm, rotated, then shrunk by 1 + d_min, d_min being the smallest norm
    among the non-centre points; sigma = scale * d_min / (1 + d_min)
    (pccnn_lib/pc/layers/KPConv.py:46-57, KPConvN.py:46-57, PCCNN.py:46-57)."""
    kp = kernel_pts_dict[str(p_dims) + "_" + str(p_num_kernel_pts)].astype(np.float32)
    dist = np.linalg.norm(kp, axis=-1).astype(np.float32)
    max_dist = np.amax(dist)
    dist, kp = dist / max_dist, kp / max_dist
    min_distance = np.amin(dist[1:])
    if kp.shape[-1] == 3:
        kp = np.dot(kp, _seeded_rotation(p_rotation_seed))
    kp = kp.astype(np.float32)
    return torch.from_numpy(kp / (1.0 + min_distance)), torch.tensor((min_distance * p_sigma_scale) / (1.0 + min_distance))


class KPConv(IConvLayer):
    """Kernel point convolution with linear correlation (pccnn_lib/pc/layers/KPConv.py:15-146).
    Buffers ``kernel_pts_`` [K, D] and ``sigma_``, parameter ``conv_weights_`` [K*Cin, Cout] keep the
    reference's names and shapes, so its state dicts load."""

    key_order_capable_ = True

    def __init__(self, p_dims, p_in_features, p_out_features, p_num_kernel_pts, p_constant_weight_var=True,
                 p_const_var_value=1.0):
        super(KPConv, self).__init__(p_dims, p_in_features, p_out_features, p_constant_weight_var,
                                     p_const_var_value)
        self.num_kernel_pts_ = p_num_kernel_pts
        self.contraction_ = "f32"       # "bf16": bf16 operands, fp32 accumulation in the [M,K*Cin] x [K*Cin,Cout] products
        kernel_pts, sigma = _kernel_point_buffers(p_dims, p_num_kernel_pts, 1.0, 15)
        self.register_buffer('kernel_pts_', kernel_pts)
        self.register_buffer('sigma_', sigma)
        self.sigma_cpu_ = None
        self._new_parameters(conv_weights_=(p_num_kernel_pts * p_in_features, p_out_features))
        self.reset_parameters()

    def reset_parameters(self):
        stdv = math.sqrt(2.0 / (self.feat_input_size_ * self.num_kernel_pts_))
        self.conv_weights_.data.normal_(0.0, stdv)

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        if self.sigma_cpu_ is None:
            self.sigma_cpu_ = self.sigma_.item()
        pts, pairs, feats = point_side(p_pc_in, p_neighborhood, p_in_features)
        geometry = (pts, feats, p_pc_out.pts_, pairs, p_neighborhood.start_ids_, p_radius, self.kernel_pts_,
                    self.sigma_cpu_)
        self._warm_up(lambda: ComputeKPConvWeightVar.apply(*geometry))
        return ComputeKPConv.apply(*geometry, self.conv_weights_, mirror_if_needed(p_neighborhood, pts),
                                   self.contraction_)


class KPConvFactory(IConvLayerFactory):
    def __init__(self, p_num_kernel_pts, p_const_var_w_init=False, p_const_var_value=1.0):
        super(KPConvFactory, self).__init__(p_num_kernel_pts, p_const_var_w_init, p_const_var_value)

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        return self._remember(KPConv(p_dims, p_in_features, p_out_features, self.num_basis_, self.conv_var_w_init_,
                                     self.const_var_value_))


class _DensityKernelPointConv(IConvLayer):
    """Shared body of the two kernel-point layers that divide by the point density: buffers ``kernel_pts_`` and
    ``sigma_``, parameter ``conv_weights_`` [K*Cin, Cout] ~ N(0, 1/(Cin*K)); the density handed to the op is
    ``pts_unnorm_pdf_ * prod(radius)``.  The layout rotation is seeded by the clock, as in the reference."""

    sigma_scale_ = 1.0
    conv_op_ = None
    weight_var_op_ = None
    key_order_capable_ = True

    def __init__(self, p_dims, p_in_features, p_out_features, p_num_kernel_pts, p_constant_weight_var=True,
                 p_const_var_value=1.0):
        super(_DensityKernelPointConv, self).__init__(p_dims, p_in_features, p_out_features, p_constant_weight_var,
                                                      p_const_var_value)
        self.num_kernel_pts_ = p_num_kernel_pts
        kernel_pts, sigma = _kernel_point_buffers(p_dims, p_num_kernel_pts, self.sigma_scale_, int(time.time()))
        self.register_buffer('kernel_pts_', kernel_pts)
        self.register_buffer('sigma_', sigma)
        self.sigma_cpu_ = None
        self._new_parameters(conv_weights_=(p_num_kernel_pts * p_in_features, p_out_features))
        self.reset_parameters()

    def reset_parameters(self):
        stdv = math.sqrt(1.0 / (self.feat_input_size_ * self.num_kernel_pts_))
        self.conv_weights_.data.normal_(0.0, stdv)

    def __compute_convolution__(self, p_pc_in, p_pc_out, p_in_features, p_radius, p_neighborhood):
        cur_pdf = density_times_volume(p_pc_in.pts_unnorm_pdf_, p_radius)
        if self.sigma_cpu_ is None:
            self.sigma_cpu_ = self.sigma_.item()
        if torch.is_grad_enabled() and cur_pdf.requires_grad:
            pts, pairs, pdf, feats = p_pc_in.pts_, p_neighborhood.neighbors_, cur_pdf, p_in_features
        else:
            pts, pairs, pdf, feats = point_side(p_pc_in, p_neighborhood, cur_pdf, p_in_features)
        geometry = (pts, pdf, feats, p_pc_out.pts_, pairs, p_neighborhood.start_ids_, p_radius, self.kernel_pts_,
                    self.sigma_cpu_)
        self._warm_up(lambda: self.weight_var_op_.apply(*geometry))
        return self.conv_op_.apply(*geometry, self.conv_weights_, mirror_if_needed(p_neighborhood, pts, pdf))


class KPConvN(_DensityKernelPointConv):
    """KPConv with density normalisation, sigma = 2 d_min / (1 + d_min) (pccnn_lib/pc/layers/KPConvN.py:13-142)."""
    sigma_scale_ = 2.0
    conv_op_ = ComputeKPConvN
    weight_var_op_ = ComputeKPConvNWeightVar


class PCCNN(_DensityKernelPointConv):
    """Gaussian kernel-point correlation with density normalisation, sigma = 0.4 d_min / (1 + d_min)
    (pccnn_lib/pc/layers/PCCNN.py:13-142)."""
    sigma_scale_ = 0.4
    conv_op_ = ComputePCCNN
    weight_var_op_ = ComputePCCNNWeightVar


class KPConvNFactory(IConvLayerFactory):
    def __init__(self, p_num_kernel_pts, p_const_var_w_init=False, p_const_var_value=1.0):
        super(KPConvNFactory, self).__init__(p_num_kernel_pts, p_const_var_w_init, p_const_var_value)

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        return self._remember(KPConvN(p_dims, p_in_features, p_out_features, self.num_basis_, self.conv_var_w_init_,
                                      self.const_var_value_))


class PCCNNFactory(IConvLayerFactory):
    def __init__(self, p_num_kernel_pts, p_const_var_w_init=False, p_const_var_value=1.0):
        super(PCCNNFactory, self).__init__(p_num_kernel_pts, p_const_var_w_init, p_const_var_value)

    def create_conv_layer(self, p_dims, p_in_features, p_out_features):
        return self._remember(PCCNN(p_dims, p_in_features, p_out_features, self.num_basis_, self.conv_var_w_init_,
                                    self.const_var_value_))
