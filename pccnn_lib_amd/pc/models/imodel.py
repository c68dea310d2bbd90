import math

from ..layers import PointConv


def _redraw_weights(layer, divisor):
    """N(0, out_constant_variance / (divisor * input features)) into the layer's weights, in place."""
    spread = math.sqrt(layer.out_constant_variance_ / (divisor * layer.feat_input_size_))
    layer.conv_weights_.data.normal_(0.0, spread)


class IModel(object):
    """Base class of a network that initialises its convolutions one after the other from the variance of their
    inputs (pccnn_lib/pc/models/IModel.py:6-27): it keeps the convolution layers in the order they were added
    (``conv_list_``) and drives, layer by layer, the warm-up state in which a layer measures its weight-variance
    statistic (the ``*_weight_var`` ops) and the re-draw of its weights from that measurement."""

    def __init__(self):
        self.conv_list_ = list()

    def _layer(self, index):
        if not 0 <= index < len(self.conv_list_):
            raise IndexError("IModel: no convolution with id %r (%d registered)" % (index, len(self.conv_list_)))
        return self.conv_list_[index]

    def add_conv(self, p_conv):
        """Register a convolution layer; its position in ``conv_list_`` is the id the other methods take."""
        self.conv_list_ += [p_conv]

    def get_num_convs(self):
        return len(self.conv_list_)

    def set_init_warmup_state(self, p_conv_id, p_w_state):
        """Switch a layer into (or out of) the state in which a forward pass measures the variance statistic of its
        projection and redraws the weights from it."""
        self._layer(p_conv_id).set_init_warmup_state(p_w_state)

    def init_variance(self, p_conv_id, p_divisor):
        """Draw the layer's weights from N(0, out_constant_variance / (p_divisor * input features)); a PointConv layer
        is also told to re-draw its projection axes on its next warm-up pass."""
        layer = self._layer(p_conv_id)
        _redraw_weights(layer, p_divisor)
        if isinstance(layer, PointConv):
            layer.init_proj_axis_ = True
