"""conv2DTranspose forward / dI / dK oracle in float64 (test infrastructure only).

Data flow restated from litenn/core/op/conv2DTranspose.py:33-47 and :50-70
(kernel is (out_ch, in_ch, KH, KW); output is (N, out_ch, OH_T, OW_T) with
OH_T / OW_T from InfoConv2D.py:45-58):

  fwd  Y  = transpose_(1,0,2,3)( K[OC, IC*KK] . im2colT(X)[IC*KK, N*OH*OW] )       (:33-35)
  dI  += transpose_(0,3,1,2)( im2row(dY)[N*IH*IW, OC*KK]
                              . transpose_(0,2,3,1)(K)[OC*KK, IC] )                 (:38-42)
  dK  += transpose_(1,0,2,3)(dY)[OC, N*OH*OW] . im2rowT(X)[N*OH*OW, IC*KK]          (:44-47)

im2colT / im2rowT are the transposed unfold (unfold2D.py:117-137): output
pixel (oh, ow) and tap (kh, kw) read input pixel ((oh + PADT - kh*d) / s,
(ow + PADL - kw*d) / s) when both divisions are exact and in range.
"""
import numpy as np

from .conv_info import info_conv2d
from .unfold import unfold_index_map, unfold_T_index_map, apply_index_map


def _geom(x_shape, k_shape, stride, dilation, padding):
    if padding not in ('valid', 'same'):
        raise ValueError('Wrong padding value, only valid or same supported for conv2DTranspose.')
    N, IC, IH, IW = x_shape
    OC, KI, KH, KW = k_shape
    if KI != IC:
        raise ValueError(f'Kernel input channels {KI} does not match input channels {IC}.')
    ci = info_conv2d(IH, IW, KH, KW, stride, dilation, padding)
    return N, IC, IH, IW, OC, KH, KW, ci


def conv2d_transpose_fwd(x, k, stride=2, dilation=1, padding='same', dtype=np.float64):
    N, IC, IH, IW, OC, KH, KW, ci = _geom(x.shape, k.shape, stride, dilation, padding)
    OH, OW = ci.OH_T, ci.OW_T
    shape, imap = unfold_T_index_map(N, IC, IH, IW, OH, OW, KH, KW, ci.PADL, ci.PADT, dilation, stride, 'CJI_NHW')
    colT = apply_index_map(x.astype(dtype), shape, imap)          # [IC*KK, N*OH*OW]
    out = k.astype(dtype).reshape(OC, -1) @ colT                  # [OC, N*OH*OW]
    return np.ascontiguousarray(out.reshape(OC, N, OH, OW).transpose(1, 0, 2, 3))


def conv2d_transpose_di(dy, k, x_shape, stride=2, dilation=1, padding='same', dtype=np.float64):
    N, IC, IH, IW, OC, KH, KW, ci = _geom(x_shape, k.shape, stride, dilation, padding)
    OH, OW = ci.OH_T, ci.OW_T
    shape, imap = unfold_index_map(N, OC, OH, OW, IH, IW, KH, KW, ci.PADL, ci.PADT, dilation, stride, 'NHW_CJI')
    row = apply_index_map(dy.astype(dtype), shape, imap)          # [N*IH*IW, OC*KK]
    kt = k.astype(dtype).transpose(0, 2, 3, 1).reshape(-1, IC)    # [OC*KK, IC]
    return np.ascontiguousarray((row @ kt).reshape(N, IH, IW, IC).transpose(0, 3, 1, 2))


def conv2d_transpose_dk(x, dy, k_shape, stride=2, dilation=1, padding='same', dtype=np.float64):
    N, IC, IH, IW, OC, KH, KW, ci = _geom(x.shape, k_shape, stride, dilation, padding)
    OH, OW = ci.OH_T, ci.OW_T
    shape, imap = unfold_T_index_map(N, IC, IH, IW, OH, OW, KH, KW, ci.PADL, ci.PADT, dilation, stride, 'NHW_CJI')
    rowT = apply_index_map(x.astype(dtype), shape, imap)          # [N*OH*OW, IC*KK]
    dy2 = dy.astype(dtype).transpose(1, 0, 2, 3).reshape(OC, -1)  # [OC, N*OH*OW]
    return (dy2 @ rowT).reshape(k_shape)


def conv2d_transpose_all(x, k, dy, stride=2, dilation=1, padding='same', dtype=np.float64):
    """(Y, dI, dK) like the reference checker's return (conv2DTranspose.py:128-…)."""
    return (conv2d_transpose_fwd(x, k, stride, dilation, padding, dtype),
            conv2d_transpose_di(dy, k, x.shape, stride, dilation, padding, dtype),
            conv2d_transpose_dk(x, dy, k.shape, stride, dilation, padding, dtype))
