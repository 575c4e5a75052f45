"""Output-size / padding arithmetic of a 2-D convolution (integers only).

Restates litenn/core/info/InfoConv2D.py:41-77.  Test infrastructure only.
"""
import math
from collections import namedtuple
from collections.abc import Iterable

ConvInfo = namedtuple('ConvInfo', 'PADL PADT PADR PADB OH OW OH_T OW_T')


def info_conv2d(H, W, KH, KW, stride, dilation, padding):
    """Paddings and output size.

    InfoConv2D.py:43-44   effective kernel  EK = (K-1)*dilation + 1
    InfoConv2D.py:48-51   'valid' -> zero pads
    InfoConv2D.py:52-58   'same'  -> left/top = floor((EK-1)/2),
                                     right/bottom = ceil((EK-1)/2)
    InfoConv2D.py:59-65   int -> all four sides; 4-sequence -> (L, T, R, B)
    InfoConv2D.py:66-67   anything else -> ValueError
    InfoConv2D.py:74-75   O = max(1, int((size + pads - EK) / stride + 1));
                          the quotient is a *float* division truncated toward
                          zero by int(), which differs from floor division
                          when the numerator is negative.
    """
    EKH = (KH - 1) * dilation + 1
    EKW = (KW - 1) * dilation + 1
    OH_T = OW_T = None
    if isinstance(padding, str) and padding == 'valid':
        PADL = PADT = PADR = PADB = 0
        OH_T = H * stride + max(EKH - stride, 0)
        OW_T = W * stride + max(EKW - stride, 0)
    elif isinstance(padding, str) and padding == 'same':
        PADL = (EKW - 1) // 2
        PADT = (EKH - 1) // 2
        PADR = EKW - 1 - PADL
        PADB = EKH - 1 - PADT
        OH_T = H * stride
        OW_T = W * stride
    elif isinstance(padding, int):   # InfoConv2D.py:59 (a bool counts as an int there too)
        PADL = PADT = PADR = PADB = padding
    elif isinstance(padding, Iterable) and not isinstance(padding, str):
        padding = tuple(int(x) for x in padding)
        if len(padding) != 4:
            raise ValueError('Invalid paddings list length.')
        PADL, PADT, PADR, PADB = padding
    else:
        raise ValueError('Invalid padding value.')
    OH = max(1, _trunc_div_plus1(H + PADT + PADB - EKH, stride))
    OW = max(1, _trunc_div_plus1(W + PADL + PADR - EKW, stride))
    return ConvInfo(PADL, PADT, PADR, PADB, OH, OW, OH_T, OW_T)


def _trunc_div_plus1(num, den):
    """int(num / den + 1) in exact integer arithmetic.

    num/den + 1 == (num + den)/den as a rational; int() truncates it toward
    zero (not toward -inf, which is what // would do for a negative value).
    """
    t = num + den
    q = abs(t) // den
    return q if t >= 0 else -q
