import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch, permuted_weights


def conv2DTranspose(input_t, kernel_t, stride=2, dilation=1, padding='same'):
    """Transposed 2-D convolution, NCHW (same call contract as conv2DTranspose.py:8-36).

     input_t    (batch, in_ch, height, width)
     kernel_t   (out_ch, in_ch, k_height, k_width)
     stride(2), dilation(1)   int
     padding    'valid' | 'same'

    The three passes are the three passes of the convolution that maps the
    (large) output back to the (small) input, with the roles swapped
    (conv2DTranspose.py:33-47): forward is that convolution's data gradient,
    dI its forward, dK its weight gradient.  They run on the same implicit-GEMM
    kernels; nothing is unfolded.  Those kernels contract over the leading
    kernel axis, i.e. they want the kernel with its two channel axes swapped:
    where they read the weights in their own permuted layout anyway, that copy
    is made straight from the kernel as stored (and kept until the kernel
    changes), and the weight gradient is written straight into the kernel's
    layout; other geometries go through an explicitly swapped kernel.
    """
    op = nc.Cacheton.get(_Conv2DTransposeOp, input_t.shape, kernel_t.shape, int(stride), int(dilation), padding)
    output_t = nn.Tensor(op.output_shape)
    output_t._set_op_name('conv2DTranspose')
    output_t._assign_gradfn(input_t, lambda O_t, dO_t: conv2DTranspose_dI_gradfn(op, input_t, kernel_t, dO_t))
    output_t._assign_gradfn(kernel_t, lambda O_t, dO_t: conv2DTranspose_dK_gradfn(op, input_t, kernel_t, dO_t))
    if op.dgrad_pw:
        wp = permuted_weights(kernel_t, op.desc, api.W_IOHW)
        launch(lambda dev, x, w, y: api.conv2d_dgrad_pw(dev, op.desc, x, w, y, 0), (input_t, 'r'), (wp, 'r'), (output_t, 'w'))
    else:
        kt = op.swapped_kernel(kernel_t)
        launch(lambda dev, x, w, y: api.conv2d_dgrad(dev, op.desc, x, w, y, 0), (input_t, 'r'), (kt, 'r'), (output_t, 'w'))
    return output_t


def conv2DTranspose_dI_gradfn(op, input_t, kernel_t, dO_t):
    """input.grad += conv2D(dO, kernel with channel axes swapped)   (conv2DTranspose.py:38-42)."""
    grad_t, beta = nc.op.accumulate_target(input_t.get_grad())
    if op.fwd_pw:
        wp = permuted_weights(kernel_t, op.desc, api.W_IOHW)
        launch(lambda dev, x, w, y: api.conv2d_fwd_pw(dev, op.desc, x, w, None, api.ACT_NONE, 0.0, y, beta),
               (dO_t, 'r'), (wp, 'r'), grad_t)
    else:
        kt = op.swapped_kernel(kernel_t)
        launch(lambda dev, x, w, y: api.conv2d_fwd(dev, op.desc, x, w, y, beta), (dO_t, 'r'), (kt, 'r'), grad_t)


def conv2DTranspose_dK_gradfn(op, input_t, kernel_t, dO_t):
    """kernel.grad += wgrad(dO, input) with its channel axes swapped back   (conv2DTranspose.py:44-47)."""
    if op.wgrad_iohw:
        grad_t, beta = nc.op.accumulate_target(kernel_t.get_grad())
        launch(lambda dev, x, dy, dw: api.conv2d_wgrad_iohw(dev, op.desc, x, dy, dw, beta), (dO_t, 'r'), (input_t, 'r'), grad_t)
        return
    dkt = nn.Tensor(op.swapped_kernel_shape)
    launch(lambda dev, x, dy, dw: api.conv2d_wgrad(dev, op.desc, x, dy, dw, 0), (dO_t, 'r'), (input_t, 'r'), (dkt, 'w'))
    nc.op.transpose(dkt, (1, 0, 2, 3), output_t=kernel_t.get_grad(), is_add_to_output=True)


class _Conv2DTransposeOp:
    """Shape plan of one transposed-convolution geometry, memoised by Cacheton
    (conv2DTranspose.py:50-70)."""

    def __init__(self, input_shape, kernel_shape, stride, dilation, padding):
        if padding not in ['valid', 'same']:
            raise ValueError('Wrong padding value, only valid or same supported for conv2DTranspose.')
        if input_shape.rank != 4 or kernel_shape.rank != 4:
            raise ValueError('conv2DTranspose expects 4-D input (N,C,H,W) and kernel (O,C,KH,KW).')
        N, IC, IH, IW = input_shape
        KO, KI, KH, KW = kernel_shape
        if KI != IC:
            raise ValueError(f'Kernel input channels {KI} does not match input channels {IC}.')
        if stride < 1 or dilation < 1:
            raise ValueError('stride and dilation must be >= 1')
        ci = nc.info.InfoConv2D(IH, IW, KH, KW, stride, dilation, padding)
        self.info = ci
        self.output_shape = nc.TensorShape((N, KO, ci.OH_T, ci.OW_T))
        self.swapped_kernel_shape = nc.TensorShape((KI, KO, KH, KW))
        # the convolution from the output image (KO channels) down to the input image (IC channels)
        self.desc = api.conv_desc(N, KO, ci.OH_T, ci.OW_T, IC, KH, KW, IH, IW, ci.PADL, ci.PADT, stride, dilation)
        # relative to that convolution the kernel is stored (C, O, KH, KW): which of its passes can take it so
        self.fwd_pw = api.conv2d_weights_plan(self.desc, api.PASS_FWD)
        self.dgrad_pw = api.conv2d_weights_plan(self.desc, api.PASS_DGRAD)
        self.wgrad_iohw = api.conv2d_weights_plan(self.desc, api.PASS_WGRAD)

    def swapped_kernel(self, kernel_t):
        kt = nn.Tensor(self.swapped_kernel_shape)
        nc.op.transpose(kernel_t, (1, 0, 2, 3), output_t=kt)
        return kt
