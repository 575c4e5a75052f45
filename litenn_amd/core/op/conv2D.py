import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch, ShallowMode


def conv2D(input_t, kernel_t, stride=1, dilation=1, padding='same'):
    """2-D cross-correlation, NCHW (same call contract as conv2D.py:9-44).

     input_t    (batch, in_ch, height, width)
     kernel_t   (out_ch, in_ch, k_height, k_width)
     stride, dilation   int
     padding    'valid' | 'same' | int | 4 ints (left, top, right, bottom)

    One implicit-GEMM launch writes the NCHW result; the reference's
    materialised im2col, its separate GeMM and the trailing transpose
    (conv2D.py:39-42) do not exist here.
    """
    op = nc.Cacheton.get(_Conv2DOp, input_t.shape, kernel_t.shape, int(stride), int(dilation), padding)
    output_t = nn.Tensor(op.output_shape)
    output_t._set_op_name('conv2D')
    output_t._assign_gradfn(input_t, lambda O_t, dO_t: conv2D_dI_gradfn(op, input_t, kernel_t, dO_t))
    output_t._assign_gradfn(kernel_t, lambda O_t, dO_t: conv2D_dK_gradfn(op, input_t, kernel_t, dO_t))
    launch(lambda dev, x, w, y: api.conv2d_fwd(dev, op.desc, x, w, y, 0), input_t, kernel_t, (output_t, 'w'))
    return output_t


def conv2D_dI_gradfn(op, input_t, kernel_t, dO_t):
    """input.grad += dgrad(dO, kernel)   (conv2D.py:46-50)."""
    grad_t, beta = nc.op.accumulate_target(input_t.get_grad())
    launch(lambda dev, dy, w, dx: api.conv2d_dgrad(dev, op.desc, dy, w, dx, beta), dO_t, kernel_t, grad_t)


def conv2D_dK_gradfn(op, input_t, kernel_t, dO_t):
    """kernel.grad += wgrad(input, dO)   (conv2D.py:52-54)."""
    grad_t, beta = nc.op.accumulate_target(kernel_t.get_grad())
    launch(lambda dev, x, dy, dw: api.conv2d_wgrad(dev, op.desc, x, dy, dw, beta), input_t, dO_t, grad_t)


class _Conv2DOp:
    """Shape plan of one convolution geometry, memoised by Cacheton
    (conv2D.py:56-73): validates channels, derives pads / output size and the
    descriptor handed to the library."""

    def __init__(self, input_shape, kernel_shape, stride, dilation, padding):
        if input_shape.rank != 4 or kernel_shape.rank != 4:
            raise ValueError('conv2D expects 4-D input (N,C,H,W) and kernel (O,C,KH,KW).')
        N, IC, IH, IW = input_shape
        KO, KI, KH, KW = kernel_shape
        if KI != IC:
            raise ValueError(f'Kernel input channels {KI} does not match tensor input channels {IC}.')
        if stride < 1 or dilation < 1:
            raise ValueError('stride and dilation must be >= 1')
        ci = nc.info.InfoConv2D(IH, IW, KH, KW, stride, dilation, padding)
        self.info = ci
        self.output_shape = nc.TensorShape((N, KO, ci.OH, ci.OW))
        self.desc = api.conv_desc(N, IC, IH, IW, KO, KH, KW, ci.OH, ci.OW, ci.PADL, ci.PADT, stride, dilation)
