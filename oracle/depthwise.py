"""depthwise_conv2D forward / dI / dK oracle in float64 (test infrastructure only).

Restated from litenn/core/op/depthwise_conv2D.py: the forward kernel
(:74-96), the data-gradient kernel (:98-124, including its exact-division
test) and the kernel gradient dK = reduce_sum_{N,OH,OW}( im2col(X) * dO )
(:44-49).  Kernel is (in_ch, KH, KW); output has in_ch channels.
"""
import numpy as np

from .conv_info import info_conv2d
from .unfold import unfold_index_map, apply_index_map


def _geom(x_shape, k_shape, stride, dilation, padding):
    if len(k_shape) != 3:
        raise ValueError('Kernel shape rank must be == 3')
    N, IC, IH, IW = x_shape
    KI, KH, KW = k_shape
    if KI != IC:
        raise ValueError(f'Kernel input channels {KI} does not match tensor input channels {IC}.')
    return N, IC, IH, IW, KH, KW, info_conv2d(IH, IW, KH, KW, stride, dilation, padding)


def depthwise_fwd(x, k, stride=1, dilation=1, padding='same', dtype=np.float64):
    N, C, IH, IW, KH, KW, ci = _geom(x.shape, k.shape, stride, dilation, padding)
    x, k = x.astype(dtype), k.astype(dtype)
    y = np.zeros((N, C, ci.OH, ci.OW), dtype)
    oh, ow = np.arange(ci.OH), np.arange(ci.OW)
    for kh in range(KH):
        ih = -ci.PADT + kh * dilation + oh * stride
        vh = (ih >= 0) & (ih < IH)
        for kw in range(KW):
            iw = -ci.PADL + kw * dilation + ow * stride
            vw = (iw >= 0) & (iw < IW)
            y[:, :, np.ix_(vh, vw)[0], np.ix_(vh, vw)[1]] += (x[:, :, ih[vh]][:, :, :, iw[vw]] *
                                                              k[None, :, kh, kw, None, None])
    return y


def depthwise_di(dy, k, x_shape, stride=1, dilation=1, padding='same', dtype=np.float64):
    N, C, IH, IW, KH, KW, ci = _geom(x_shape, k.shape, stride, dilation, padding)
    dy, k = dy.astype(dtype), k.astype(dtype)
    dx = np.zeros((N, C, IH, IW), dtype)
    ih, iw = np.arange(IH), np.arange(IW)
    for kh in range(KH):
        nh = ci.PADT + ih - kh * dilation
        oh = np.floor_divide(nh, stride)
        vh = (nh >= 0) & (oh * stride == nh) & (oh < ci.OH)
        for kw in range(KW):
            nw = ci.PADL + iw - kw * dilation
            ow = np.floor_divide(nw, stride)
            vw = (nw >= 0) & (ow * stride == nw) & (ow < ci.OW)
            dx[:, :, np.ix_(vh, vw)[0], np.ix_(vh, vw)[1]] += (dy[:, :, oh[vh]][:, :, :, ow[vw]] *
                                                               k[None, :, kh, kw, None, None])
    return dx


def depthwise_dk(x, dy, k_shape, stride=1, dilation=1, padding='same', dtype=np.float64):
    N, C, IH, IW, KH, KW, ci = _geom(x.shape, k_shape, stride, dilation, padding)
    shape, imap = unfold_index_map(N, C, IH, IW, ci.OH, ci.OW, KH, KW, ci.PADL, ci.PADT, dilation, stride, 'CJI_NHW')
    col = apply_index_map(x.astype(dtype), shape, imap).reshape(C, KH, KW, -1)      # [C, KH, KW, N*OH*OW]
    dy2 = dy.astype(dtype).transpose(1, 0, 2, 3).reshape(C, 1, 1, -1)
    return (col * dy2).sum(-1)


def depthwise_all(x, k, dy, stride=1, dilation=1, padding='same', dtype=np.float64):
    return (depthwise_fwd(x, k, stride, dilation, padding, dtype),
            depthwise_di(dy, k, x.shape, stride, dilation, padding, dtype),
            depthwise_dk(x, dy, k.shape, stride, dilation, padding, dtype))
