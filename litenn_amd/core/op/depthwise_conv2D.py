import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch


def depthwise_conv2D(input_t, kernel_t, stride=1, dilation=1, padding='same'):
    """Depthwise 2-D convolution, NCHW (same call contract as depthwise_conv2D.py:9-39).

     input_t    (batch, in_ch, height, width)
     kernel_t   (in_ch, k_height, k_width)
     stride, dilation   int
     padding    'valid' | 'same' | int | 4 ints (left, top, right, bottom)

    No contraction over channels: three bandwidth-bound kernels (forward, data
    gradient, kernel gradient).  The kernel gradient sums X * dO over batch and
    pixels per tap directly instead of materialising the unfolded input
    (depthwise_conv2D.py:44-49).
    """
    op = nc.Cacheton.get(_DepthwiseConv2DOp, input_t.shape, kernel_t.shape, int(stride), int(dilation), padding)
    output_t = nn.Tensor(op.output_shape)
    output_t._set_op_name('depthwise_conv2D')
    output_t._assign_gradfn(input_t, lambda O_t, dO_t: depthwise_dI_gradfn(op, input_t, kernel_t, dO_t))
    output_t._assign_gradfn(kernel_t, lambda O_t, dO_t: depthwise_dK_gradfn(op, input_t, kernel_t, dO_t))
    launch(lambda dev, x, k, y: api.depthwise_conv2d_fwd(dev, op.desc, x, k, y, 0), (input_t, 'r'), (kernel_t, 'r'), (output_t, 'w'))
    return output_t


def depthwise_dI_gradfn(op, input_t, kernel_t, dO_t):
    grad_t, beta = nc.op.accumulate_target(input_t.get_grad())
    launch(lambda dev, dy, k, dx: api.depthwise_conv2d_dgrad(dev, op.desc, dy, k, dx, beta), (dO_t, 'r'), (kernel_t, 'r'), grad_t)


def depthwise_dK_gradfn(op, input_t, kernel_t, dO_t):
    grad_t, beta = nc.op.accumulate_target(kernel_t.get_grad())
    launch(lambda dev, x, dy, dk: api.depthwise_conv2d_wgrad(dev, op.desc, x, dy, dk, beta), (input_t, 'r'), (dO_t, 'r'), grad_t)


class _DepthwiseConv2DOp:
    """Shape plan, memoised by Cacheton (depthwise_conv2D.py:51-66)."""

    def __init__(self, input_shape, kernel_shape, stride, dilation, padding):
        if kernel_shape.rank != 3:
            raise ValueError('Kernel shape rank must be == 3')
        if input_shape.rank != 4:
            raise ValueError('depthwise_conv2D expects a 4-D input (N,C,H,W).')
        N, IC, IH, IW = input_shape
        KI, KH, KW = kernel_shape
        if KI != IC:
            raise ValueError(f'Kernel input channels {KI} does not match tensor input channels {IC}.')
        if stride < 1 or dilation < 1:
            raise ValueError('stride and dilation must be >= 1')
        ci = nc.info.InfoConv2D(IH, IW, KH, KW, stride, dilation, padding)
        self.info = ci
        self.output_shape = nc.TensorShape((N, IC, ci.OH, ci.OW))
        self.desc = api.conv_desc(N, IC, IH, IW, IC, KH, KW, ci.OH, ci.OW, ci.PADL, ci.PADT, stride, dilation)
