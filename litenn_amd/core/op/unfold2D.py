import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch

_ORDERS = {'CJI_NHW': 0, 'NHW_CJI': 1}


def unfold2D(input_t, N, C, H, W, OH, OW, KH, KW, PADL, PADT, DILATION, STRIDE, sshape, is_transpose,
             input_data_format='NCHW', output_t=None, is_add_to_output=False):
    """Materialised im2col ('CJI_NHW'), im2row ('NHW_CJI') or, with
    is_transpose, the transposed im2row used for input gradients
    (unfold2D.py:6-48).  conv2D itself never calls this - its kernels gather on
    the fly - but the op is kept for code written against it and as the
    observable form of the gather index arithmetic.  Only NCHW input and the
    two layouts the reference's conv2D uses are provided.  No gradient."""
    is_add_to_output = False if output_t is None else is_add_to_output
    if input_data_format != 'NCHW':
        raise ValueError(f'Unsupported input_data_format {input_data_format}.')
    order = _ORDERS.get(sshape.upper())
    if order is None:
        raise ValueError(f'Unsupported sshape {sshape}. Provided: {list(_ORDERS)}')
    N, C, H, W, OH, OW, KH, KW, PADL, PADT, DILATION, STRIDE = (
        int(x) for x in (N, C, H, W, OH, OW, KH, KW, PADL, PADT, DILATION, STRIDE))
    rows, cols = (C * KH * KW, N * OH * OW) if order == 0 else (N * OH * OW, C * KH * KW)
    if input_t.shape.size != N * C * H * W:
        raise ValueError(f'input_t must have size {N*C*H*W}')
    if output_t is None:
        output_t = nn.Tensor((rows, cols))
        output_t._set_op_name('unfold2D')
    elif output_t.shape.size != rows * cols:
        raise ValueError(f'output_t must have size {rows*cols}')
    beta = 1 if is_add_to_output else 0
    out_arg = output_t if is_add_to_output else (output_t, 'w')
    launch(lambda dev, i, o: api.unfold2d(dev, N, C, H, W, OH, OW, KH, KW, PADL, PADT, DILATION, STRIDE, order,
                                          bool(is_transpose), i, o, beta), (input_t, 'r'), out_arg)
    return output_t
