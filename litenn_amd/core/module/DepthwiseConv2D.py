import litenn_amd as nn
import litenn_amd.core as nc


class DepthwiseConv2D(nn.Module):
    """Depthwise convolution layer (same constructor and forward as module/DepthwiseConv2D.py).

     in_ch, kernel_size   ints
     stride(1) dilation(1)
     padding('same')   'valid' | 'same' | int | 4 ints (left, top, right, bottom)
     use_bias(True)
     depthwise_initializer   default: hint value or nn.initializer.GlorotUniform()
     pointwise_initializer   accepted and unused, as in the reference's signature
     bias_initializer        default: nn.initializer.Scalar(0.0)
    """

    def __init__(self, in_ch, kernel_size, stride=1, dilation=1, padding='same', use_bias=True,
                 depthwise_initializer=None, pointwise_initializer=None, bias_initializer=None):
        self.in_ch, self.kernel_size = in_ch, kernel_size
        self.stride, self.padding, self.dilation, self.use_bias = stride, padding, dilation, use_bias
        kernel_initializer = depthwise_initializer
        if kernel_initializer is None:
            kernel_initializer = nc.Cacheton.get_var('DepthwiseConv2D_default_depthwise_initializer')
        if kernel_initializer is None:
            kernel_initializer = nn.initializer.GlorotUniform()
        if kernel_initializer.has_fan_in() and kernel_initializer.fan_in is None:
            kernel_initializer.fan_in = in_ch * kernel_size * kernel_size
        if kernel_initializer.has_fan_out() and kernel_initializer.fan_out is None:
            kernel_initializer.fan_out = 0
        self.depthwise_initializer = kernel_initializer
        self.kernel = nn.Tensor((in_ch, kernel_size, kernel_size), init=kernel_initializer)
        self.bias = None
        if use_bias:
            if bias_initializer is None:
                bias_initializer = nn.initializer.Scalar(0.0)
            self.bias_initializer = bias_initializer
            self.bias = nn.Tensor((in_ch,), init=bias_initializer)
        super().__init__(saveables=['kernel', 'bias'])

    def forward(self, x, **kwargs):
        x = nn.depthwise_conv2D(x, self.kernel, self.stride, self.dilation, padding=self.padding)
        if self.use_bias:
            x = x + self.bias.reshape((1, -1, 1, 1))
        return x

    def __str__(self): return f'{self.__class__.__name__} : in_ch:{self.in_ch} '
    __repr__ = __str__


def hint_DepthwiseConv2D_default_depthwise_initializer(depthwise_initializer):
    """Default kernel initializer of later DepthwiseConv2D layers, until nn.cleanup()."""
    if not isinstance(depthwise_initializer, nn.initializer.Initializer):
        raise ValueError('depthwise_initializer should be class of nn.initializer.*')
    nc.Cacheton.set_var('DepthwiseConv2D_default_depthwise_initializer', depthwise_initializer)
