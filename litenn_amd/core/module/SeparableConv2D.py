import litenn_amd as nn
import litenn_amd.core as nc


class SeparableConv2D(nn.Module):
    """Depthwise convolution followed by a 1x1 convolution (same constructor and forward as
    module/SeparableConv2D.py:6-82).

     in_ch, out_ch, kernel_size   ints
     stride(1) dilation(1)
     padding('same')   'valid' | 'same' | int | 4 ints (left, top, right, bottom)
     use_bias(True)
     depthwise_initializer, pointwise_initializer   default: hint value or nn.initializer.GlorotUniform()
     bias_initializer     default: nn.initializer.Scalar(0.0)
    """

    def __init__(self, in_ch, out_ch, kernel_size, stride=1, dilation=1, padding='same', use_bias=True,
                 depthwise_initializer=None, pointwise_initializer=None, bias_initializer=None):
        self.in_ch, self.out_ch, self.kernel_size = in_ch, out_ch, kernel_size
        self.stride, self.padding, self.dilation, self.use_bias = stride, padding, dilation, use_bias
        if depthwise_initializer is None:
            depthwise_initializer = nc.Cacheton.get_var('SeparableConv2D_default_depthwise_initializer')
        if depthwise_initializer is None:
            depthwise_initializer = nn.initializer.GlorotUniform()
        if depthwise_initializer.has_fan_in() and depthwise_initializer.fan_in is None:
            depthwise_initializer.fan_in = in_ch * kernel_size * kernel_size
        if depthwise_initializer.has_fan_out() and depthwise_initializer.fan_out is None:
            depthwise_initializer.fan_out = 0
        self.depthwise_initializer = depthwise_initializer
        self.depthwise_kernel = nn.Tensor((in_ch, kernel_size, kernel_size), init=depthwise_initializer)
        if pointwise_initializer is None:
            pointwise_initializer = nc.Cacheton.get_var('SeparableConv2D_default_pointwise_initializer')
        if pointwise_initializer is None:
            pointwise_initializer = nn.initializer.GlorotUniform()
        if pointwise_initializer.has_fan_in() and pointwise_initializer.fan_in is None:
            pointwise_initializer.fan_in = in_ch
        if pointwise_initializer.has_fan_out() and pointwise_initializer.fan_out is None:
            pointwise_initializer.fan_out = out_ch
        self.pointwise_initializer = pointwise_initializer
        self.pointwise_kernel = nn.Tensor((out_ch, in_ch, 1, 1), init=pointwise_initializer)
        self.bias = None
        if use_bias:
            if bias_initializer is None:
                bias_initializer = nn.initializer.Scalar(0.0)
            self.bias_initializer = bias_initializer
            self.bias = nn.Tensor((out_ch,), init=bias_initializer)
        super().__init__(saveables=['depthwise_kernel', 'pointwise_kernel', 'bias'])

    def forward(self, x, **kwargs):
        x = nn.depthwise_conv2D(x, self.depthwise_kernel, self.stride, self.dilation, padding=self.padding)
        if self.use_bias:
            # the 1x1 convolution with the bias add in its epilogue (module/SeparableConv2D.py:77-81)
            return nc.op.conv2D_bias_act(x, self.pointwise_kernel, self.bias, 1, 1, 'valid')
        return nn.conv2D(x, self.pointwise_kernel, 1, 1, padding='valid')

    def __str__(self): return f'{self.__class__.__name__} : in_ch:{self.in_ch} out_ch:{self.out_ch} '
    __repr__ = __str__


def hint_SeparableConv2D_default_depthwise_initializer(depthwise_initializer):
    """Default depthwise initializer of later SeparableConv2D layers, until nn.cleanup()."""
    if not isinstance(depthwise_initializer, nn.initializer.Initializer):
        raise ValueError('depthwise_initializer should be class of nn.initializer.*')
    nc.Cacheton.set_var('SeparableConv2D_default_depthwise_initializer', depthwise_initializer)


def hint_SeparableConv2D_default_pointwise_initializer(pointwise_initializer):
    """Default pointwise initializer of later SeparableConv2D layers, until nn.cleanup()."""
    if not isinstance(pointwise_initializer, nn.initializer.Initializer):
        raise ValueError('pointwise_initializer should be class of nn.initializer.*')
    nc.Cacheton.set_var('SeparableConv2D_default_pointwise_initializer', pointwise_initializer)
