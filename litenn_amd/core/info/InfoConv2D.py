from collections.abc import Iterable


class InfoConv2D:
    """Padding and output-size arithmetic of a 2-D convolution, integers only
    (same results as InfoConv2D.py:41-77).

     H, W, KH, KW, stride, dilation   ints
     padding   'valid' | 'same' | int (all sides) | 4 ints (left, top, right, bottom)

    result: .PADL .PADR .PADT .PADB .OH .OW and, for 'valid'/'same' only,
    .OH_T .OW_T (output size of the transposed convolution), else None.
    Raises ValueError for anything else.
    """
    __slots__ = ['PADL', 'PADR', 'PADT', 'PADB', 'OH', 'OW', 'OH_T', 'OW_T']

    def __init__(self, H, W, KH, KW, stride, dilation, padding):
        ekh = (KH - 1) * dilation + 1
        ekw = (KW - 1) * dilation + 1
        self.OH_T = self.OW_T = None
        if isinstance(padding, str):
            if padding == 'valid':
                self.PADL = self.PADT = self.PADR = self.PADB = 0
                self.OH_T = H * stride + max(ekh - stride, 0)
                self.OW_T = W * stride + max(ekw - stride, 0)
            elif padding == 'same':
                # the odd pad, if any, goes to the right / bottom
                self.PADL, self.PADT = (ekw - 1) // 2, (ekh - 1) // 2
                self.PADR, self.PADB = ekw - 1 - self.PADL, ekh - 1 - self.PADT
                self.OH_T, self.OW_T = H * stride, W * stride
            else:
                raise ValueError('Invalid padding value.')
        elif isinstance(padding, int):
            self.PADL = self.PADT = self.PADR = self.PADB = padding
        elif isinstance(padding, Iterable):
            pads = tuple(int(x) for x in padding)
            if len(pads) != 4:
                raise ValueError('Invalid paddings list length.')
            self.PADL, self.PADT, self.PADR, self.PADB = pads
        else:
            raise ValueError('Invalid padding value.')
        self.OH = max(1, _quotient_plus_one(H + self.PADT + self.PADB - ekh, stride))
        self.OW = max(1, _quotient_plus_one(W + self.PADL + self.PADR - ekw, stride))


def _quotient_plus_one(num, den):
    """num/den + 1 truncated toward zero, exactly (the reference evaluates
    int(num / den + 1) in floating point, InfoConv2D.py:74-75)."""
    t = num + den
    return t // den if t >= 0 else -((-t) // den)
