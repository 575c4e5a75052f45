import litenn_amd as nn
import litenn_amd.core as nc


class Dense(nn.Module):
    """Fully connected layer x(...,in_ch) @ weight(in_ch,out_ch) + bias
    (same constructor and forward as module/Dense.py:5-48)."""

    def __init__(self, in_ch, out_ch, use_bias=True, weight_initializer=None, bias_initializer=None):
        self.in_ch, self.out_ch, self.use_bias = in_ch, out_ch, use_bias
        if weight_initializer is None:
            weight_initializer = nc.Cacheton.get_var('Dense_default_weight_initializer')
        if weight_initializer is None:
            weight_initializer = nn.initializer.GlorotUniform()
        if weight_initializer.has_fan_in() and weight_initializer.fan_in is None:
            weight_initializer.fan_in = in_ch
        if weight_initializer.has_fan_out() and weight_initializer.fan_out is None:
            weight_initializer.fan_out = out_ch
        self.weight = nn.Tensor((in_ch, out_ch), init=weight_initializer)
        self.bias = None
        if use_bias:
            if bias_initializer is None:
                bias_initializer = nn.initializer.Scalar(0.0)
            self.bias_initializer = bias_initializer
            self.bias = nn.Tensor((out_ch,), init=bias_initializer)
        super().__init__(saveables=['weight', 'bias'])

    def forward(self, x, **kwargs):
        # nn.matmul(x, weight) + bias (module/Dense.py:44-48) with the bias added in the product's epilogue
        if self.use_bias and x.shape.rank == 2:
            return nc.op.matmul_bias_act(x, self.weight, self.bias)
        x = nn.matmul(x, self.weight)
        if self.use_bias:
            x = x + self.bias
        return x

    def __str__(self): return f'{self.__class__.__name__} : in_ch:{self.in_ch} out_ch:{self.out_ch} '
    __repr__ = __str__


def hint_Dense_default_weight_initializer(weight_initializer):
    """Default weight initializer of later Dense layers, until nn.cleanup()."""
    if not isinstance(weight_initializer, nn.initializer.Initializer):
        raise ValueError('weight_initializer should be class of nn.initializer.*')
    nc.Cacheton.set_var('Dense_default_weight_initializer', weight_initializer)
