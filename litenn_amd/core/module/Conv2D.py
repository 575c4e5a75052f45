import litenn_amd as nn
import litenn_amd.core as nc


class Conv2D(nn.Module):
    """2-D convolution layer (same constructor and forward as module/Conv2D.py:6-62).

     in_ch, out_ch, kernel_size   ints
     stride(1) dilation(1)
     padding('same')   'valid' | 'same' | int | 4 ints (left, top, right, bottom)
     use_bias(True)
     kernel_initializer   default: hint value or nn.initializer.GlorotUniform()
     bias_initializer     default: nn.initializer.Scalar(0.0)
    """

    def __init__(self, in_ch, out_ch, kernel_size, stride=1, dilation=1, padding='same', use_bias=True,
                 kernel_initializer=None, bias_initializer=None):
        self.in_ch, self.out_ch, self.kernel_size = in_ch, out_ch, kernel_size
        self.stride, self.padding, self.dilation, self.use_bias = stride, padding, dilation, use_bias
        if kernel_initializer is None:
            kernel_initializer = nc.Cacheton.get_var('Conv2D_default_kernel_initializer')
        if kernel_initializer is None:
            kernel_initializer = nn.initializer.GlorotUniform()
        if kernel_initializer.has_fan_in() and kernel_initializer.fan_in is None:
            kernel_initializer.fan_in = in_ch * kernel_size * kernel_size
        if kernel_initializer.has_fan_out() and kernel_initializer.fan_out is None:
            kernel_initializer.fan_out = out_ch * kernel_size * kernel_size
        self.kernel_initializer = kernel_initializer
        self.kernel = nn.Tensor((out_ch, in_ch, kernel_size, kernel_size), init=kernel_initializer)
        self.bias = None
        if use_bias:
            if bias_initializer is None:
                bias_initializer = nn.initializer.Scalar(0.0)
            self.bias_initializer = bias_initializer
            self.bias = nn.Tensor((out_ch,), init=bias_initializer)
        super().__init__(saveables=['kernel', 'bias'])

    def forward(self, x, **kwargs):
        if self.use_bias:
            # conv2D followed by x + bias.reshape((1,-1,1,1)) (module/Conv2D.py:59-62), the add done in the
            # convolution's epilogue: same values, same gradients, one pass over the output instead of two
            return nc.op.conv2D_bias_act(x, self.kernel, self.bias, self.stride, self.dilation, self.padding)
        return nn.conv2D(x, self.kernel, self.stride, self.dilation, padding=self.padding)

    def __str__(self): return f'{self.__class__.__name__} : in_ch:{self.in_ch} out_ch:{self.out_ch} '
    __repr__ = __str__


def hint_Conv2D_default_kernel_initializer(kernel_initializer):
    """Default kernel initializer of later Conv2D layers, until nn.cleanup()."""
    if not isinstance(kernel_initializer, nn.initializer.Initializer):
        raise ValueError('kernel_initializer should be class of nn.initializer.*')
    nc.Cacheton.set_var('Conv2D_default_kernel_initializer', kernel_initializer)
