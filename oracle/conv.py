"""conv2D forward / dX / dW oracle in float64 (test infrastructure only).

Data flow restated from litenn/core/op/conv2D.py:39-54:

  fwd  Y  = transpose_(1,0,2,3)( W[O,CKK] . im2col(X)[CKK,P] )      (:39-42)
  dX  += transpose_(0,3,1,2)( im2rowT(dY)[N*IH*IW, O*KK]
                              . transpose_(0,2,3,1)(W)[O*KK, C] )    (:46-50)
  dW  += transpose_(1,0,2,3)(dY)[O,P] . im2row(X)[P,CKK]            (:52-54)

The maths these compute is the cross-correlation checked by the reference's
own numpy checker (conv2D.py:128-219):
  Y[n,o,oh,ow] = sum_{c,kh,kw} X[n,c,oh*s-PT+kh*d, ow*s-PL+kw*d] W[o,c,kh,kw]
with out-of-range X taken as zero, and dX / dW its two adjoints.
"""
import numpy as np

from .conv_info import info_conv2d
from .unfold import unfold_index_map, unfold_T_index_map, apply_index_map


def _geom(x_shape, w_shape, stride, dilation, padding):
    N, C, IH, IW = x_shape
    O, KI, KH, KW = w_shape
    if KI != C:
        raise ValueError(f'Kernel input channels {KI} does not match tensor input channels {C}.')
    ci = info_conv2d(IH, IW, KH, KW, stride, dilation, padding)
    return N, C, IH, IW, O, KH, KW, ci


def conv2d_fwd(x, w, stride=1, dilation=1, padding='same', dtype=np.float64):
    N, C, IH, IW, O, KH, KW, ci = _geom(x.shape, w.shape, stride, dilation, padding)
    shape, imap = unfold_index_map(N, C, IH, IW, ci.OH, ci.OW, KH, KW, ci.PADL, ci.PADT,
                                   dilation, stride, 'CJI_NHW')
    col = apply_index_map(x.astype(dtype), shape, imap)            # [CKK, P]
    out = w.astype(dtype).reshape(O, -1) @ col                     # [O, P]
    return np.ascontiguousarray(out.reshape(O, N, ci.OH, ci.OW).transpose(1, 0, 2, 3))


def conv2d_dx(dy, w, x_shape, stride=1, dilation=1, padding='same', dtype=np.float64):
    N, C, IH, IW, O, KH, KW, ci = _geom(x_shape, w.shape, stride, dilation, padding)
    shape, imap = unfold_T_index_map(N, O, ci.OH, ci.OW, IH, IW, KH, KW, ci.PADL, ci.PADT,
                                     dilation, stride, 'NHW_CJI')
    rowT = apply_index_map(dy.astype(dtype), shape, imap)          # [N*IH*IW, O*KK]
    wt = w.astype(dtype).transpose(0, 2, 3, 1).reshape(-1, C)      # [O*KK, C]
    out = rowT @ wt                                                # [N*IH*IW, C]
    return np.ascontiguousarray(out.reshape(N, IH, IW, C).transpose(0, 3, 1, 2))


def conv2d_dw(x, dy, w_shape, stride=1, dilation=1, padding='same', dtype=np.float64):
    N, C, IH, IW, O, KH, KW, ci = _geom(x.shape, w_shape, stride, dilation, padding)
    shape, imap = unfold_index_map(N, C, IH, IW, ci.OH, ci.OW, KH, KW, ci.PADL, ci.PADT,
                                   dilation, stride, 'NHW_CJI')
    row = apply_index_map(x.astype(dtype), shape, imap)            # [P, CKK]
    dy2 = dy.astype(dtype).transpose(1, 0, 2, 3).reshape(O, -1)    # [O, P]
    return (dy2 @ row).reshape(w_shape)


def conv2d_all(x, w, dy, stride=1, dilation=1, padding='same', dtype=np.float64):
    """(Y, dX, dW) like the reference checker's return (conv2D.py:219)."""
    return (conv2d_fwd(x, w, stride, dilation, padding, dtype),
            conv2d_dx(dy, w, x.shape, stride, dilation, padding, dtype),
            conv2d_dw(x, dy, w.shape, stride, dilation, padding, dtype))
