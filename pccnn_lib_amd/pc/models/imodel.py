import math

from ..layers import PointConv


class IModel(object):
    """Base class of a network that initialises its convolutions one after the other from the variance of their
    inputs (pccnn_lib/pc/models/IModel.py:6-27): it keeps the convolution layers in the order they were added
    (``conv_list_``) and drives, layer by layer, the warm-up state in which a layer measures its weight-variance
    statistic (the ``*_weight_var`` ops) and the re-draw of its weights from that measurement."""

    def __init__(self):
        self.conv_list_ = []

    def add_conv(self, p_conv):
        """Register a convolution layer; its index in ``conv_list_`` is the id the other methods take."""
        self.conv_list_.append(p_conv)

    def get_num_convs(self):
        return len(self.conv_list_)

    def set_init_warmup_state(self, p_conv_id, p_w_state):
        """Switch layer ``p_conv_id`` into (or out of) the state in which a forward pass only accumulates the
        variance statistic of its projection."""
        self.conv_list_[p_conv_id].set_init_warmup_state(p_w_state)

    def init_variance(self, p_conv_id, p_divisor):
        """Draw the weights of layer ``p_conv_id`` from N(0, out_constant_variance / (p_divisor * input features));
        a PointConv layer is also told to re-draw its projection axes on its next warm-up pass."""
        conv = self.conv_list_[p_conv_id]
        fan = p_divisor * conv.feat_input_size_
        conv.conv_weights_.data.normal_(0.0, math.sqrt(conv.out_constant_variance_ / fan))
        if isinstance(conv, PointConv):
            conv.init_proj_axis_ = True
