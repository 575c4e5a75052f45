import litenn_amd as nn
import litenn_amd.core as nc
from ..backward import after_gradfns_of_tensor, current_sweep
from ..hip import api, launch, permuted_weights, ShallowMode


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
    if op.fwd_pw:
        launch(lambda dev, x, wp, y: api.conv2d_fwd_pw(dev, op.desc, x, wp, None, api.ACT_NONE, 0.0, y, 0),
               (input_t, 'r'), (permuted_weights(kernel_t, op.desc), 'r'), (output_t, 'w'))
    else:
        launch(lambda dev, x, w, y: api.conv2d_fwd(dev, op.desc, x, w, y, 0), (input_t, 'r'), (kernel_t, 'r'), (output_t, 'w'))
    return output_t


def conv2D_bias_act(input_t, kernel_t, bias_t=None, stride=1, dilation=1, padding='same', leaky_relu_alpha=None):
    """leaky_relu(conv2D(input, kernel) + bias.reshape(1,-1,1,1), alpha) in one launch.

    The three steps as a layer writes them (module/Conv2D.py:59-62 followed by
    element_wise_op.py:216-222) cost two extra read+write passes over the
    output; here the convolution's epilogue adds bias[o] and applies the
    activation to the fp32 accumulator before its only store, which gives the
    same bits.  bias_t (out_ch,) and leaky_relu_alpha are optional;
    alpha must be > 0 (the backward pass reads the sign of the pre-activation
    off the output).  Gradients: input and kernel as conv2D, bias the sum of
    the pre-activation gradient over batch and pixels, each accumulated.
    """
    op = nc.Cacheton.get(_Conv2DOp, input_t.shape, kernel_t.shape, int(stride), int(dilation), padding)
    if bias_t is not None and tuple(bias_t.shape) != (kernel_t.shape[0],):
        raise ValueError(f'bias shape {tuple(bias_t.shape)} does not match {kernel_t.shape[0]} output channels')
    if leaky_relu_alpha is not None and not leaky_relu_alpha > 0:
        raise ValueError('leaky_relu_alpha must be > 0 for the fused form')
    act = api.ACT_NONE if leaky_relu_alpha is None else api.ACT_LEAKY_RELU
    alpha = 0.0 if leaky_relu_alpha is None else float(leaky_relu_alpha)
    output_t = nn.Tensor(op.output_shape)
    output_t._set_op_name('conv2D_bias_act')
    epi = _EpilogueGrad(act, alpha)
    # the bias comes first: when its gradient is wanted, the one pass that forms the pre-activation gradient also
    # sums it per channel
    if bias_t is not None:
        output_t._assign_gradfn(bias_t, lambda O_t, dO_t: epi.bias(O_t, dO_t, bias_t))
    output_t._assign_gradfn(input_t, lambda O_t, dO_t: conv2D_dI_gradfn(op, input_t, kernel_t, epi.pre(O_t, dO_t)))
    output_t._assign_gradfn(kernel_t, lambda O_t, dO_t: conv2D_dK_gradfn(op, input_t, kernel_t, epi.pre(O_t, dO_t)))
    args = [(input_t, 'r'), (permuted_weights(kernel_t, op.desc), 'r') if op.fwd_pw else (kernel_t, 'r')]
    if bias_t is not None:
        args.append((bias_t, 'r'))

    def run(dev, x, w, *rest):
        b, y = (rest[0], rest[1]) if bias_t is not None else (None, rest[0])
        if op.fwd_pw:
            api.conv2d_fwd_pw(dev, op.desc, x, w, b, act, alpha, y, 0)
        else:
            api.conv2d_fwd_bias_act(dev, op.desc, x, w, b, act, alpha, y)
    launch(run, *args, (output_t, 'w'))
    return output_t


class _EpilogueGrad:
    """Backward of the fused epilogue, shared by the gradient functions of one conv2D_bias_act result.

    pre(): dO * f'(pre-activation), formed once per backward pass.  For leaky ReLU with alpha > 0 the output has
    the sign of the pre-activation, so f' is read off the output.
    bias(): bias.grad[o] += sum of that over batch and pixels (dual_wise_op.py:110-130 for the broadcast
    operand) - in the same launch as pre() when it runs first, which it does whenever the bias gradient is
    wanted at all."""

    def __init__(self, act, alpha, dims=None):
        self.act, self.alpha = act, alpha
        # (batch, channels, elements per channel plane) of the output: NCHW by default; a dense layer's (rows, out_ch)
        # is the same with planes of one element
        self.dims = dims if dims is not None else (lambda shape: (shape[0], shape[1], shape[2] * shape[3]))
        self.key, self.value = None, None      # key: (backward sweep, the dO tensor the value was formed from)

    def _drop(self):
        self.key, self.value = None, None

    def _cached(self, dO_t):
        sweep = current_sweep()
        return (sweep is not None and self.key is not None and self.key[0] == sweep and self.key[1] is dO_t)

    def _run(self, O_t, dO_t, want_pre, bias_grad):
        N, O, HW = self.dims(tuple(dO_t.shape))
        pre = None
        if want_pre:
            pre = nn.Tensor(dO_t.shape)
            self.value = pre
            # valid for the gradient functions of this output in this sweep only: they run one after the other, and
            # the tensor is let go when the last of them has
            if current_sweep() is not None:
                self.key = (current_sweep(), dO_t)
                after_gradfns_of_tensor(self._drop)
        args = [O_t, dO_t]
        if pre is not None:
            args.append((pre, 'w'))
        beta = 0
        if bias_grad is not None:
            target, beta = nc.op.accumulate_target(bias_grad)
            args.append(target)

        def run(dev, y, dy, *outs):
            outs = list(outs)
            dpre = outs.pop(0) if pre is not None else None
            dbias = outs.pop(0) if bias_grad is not None else None
            api.bias_act_bwd(dev, N, O, HW, y, dy, self.act, self.alpha, dpre, dbias, beta)
        launch(run, *args)

    def pre(self, O_t, dO_t):
        if self.act == api.ACT_NONE:
            return dO_t
        if self._cached(dO_t):
            return self.value
        self._run(O_t, dO_t, True, None)
        value = self.value
        if current_sweep() is None:
            self._drop()
        return value

    def bias(self, O_t, dO_t, bias_t):
        self._run(O_t, dO_t, self.act != api.ACT_NONE and not self._cached(dO_t), bias_t.get_grad())
        if current_sweep() is None:
            self._drop()


def conv2D_dI_gradfn(op, input_t, kernel_t, dO_t):
    """input.grad += dgrad(dO, kernel)   (conv2D.py:46-50)."""
    grad_t, beta = nc.op.accumulate_target(input_t.get_grad())
    if op.dgrad_pw:
        launch(lambda dev, dy, wp, dx: api.conv2d_dgrad_pw(dev, op.desc, dy, wp, dx, beta),
               (dO_t, 'r'), (permuted_weights(kernel_t, op.desc), 'r'), grad_t)
    else:
        launch(lambda dev, dy, w, dx: api.conv2d_dgrad(dev, op.desc, dy, w, dx, beta), (dO_t, 'r'), (kernel_t, 'r'), grad_t)


def conv2D_dK_gradfn(op, input_t, kernel_t, dO_t):
    """kernel.grad += wgrad(input, dO)   (conv2D.py:52-54)."""
    grad_t, beta = nc.op.accumulate_target(kernel_t.get_grad())
    launch(lambda dev, x, dy, dw: api.conv2d_wgrad(dev, op.desc, x, dy, dw, beta), (input_t, 'r'), (dO_t, 'r'), grad_t)


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
        # whether this geometry's forward / data-gradient kernels read the weights in their permuted layout, of
        # which one cached copy then serves both passes until the weights change
        self.fwd_pw = api.conv2d_weights_plan(self.desc, api.PASS_FWD)
        self.dgrad_pw = api.conv2d_weights_plan(self.desc, api.PASS_DGRAD)
