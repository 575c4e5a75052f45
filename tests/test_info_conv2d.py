"""The product's InfoConv2D (litenn_amd.core.info, restating InfoConv2D.py:41-77) compared field for field with
the pinned oracle over a grid that covers what the kernels never see through output shapes alone: negative
numerators (the quotient truncates toward zero, then clamps to 1), asymmetric 4-tuples in every container type,
the transposed sizes OH_T / OW_T, and the error paths."""
import itertools

import numpy as np
import pytest

from litenn_amd.core.info import InfoConv2D
from oracle import info_conv2d

FIELDS = ('PADL', 'PADT', 'PADR', 'PADB', 'OH', 'OW', 'OH_T', 'OW_T')


def _same(H, W, KH, KW, s, d, padding):
    got = InfoConv2D(H, W, KH, KW, s, d, padding)
    ref = info_conv2d(H, W, KH, KW, s, d, padding)
    for f in FIELDS:
        g, r = getattr(got, f), getattr(ref, f)
        assert g == r and type(g) is type(r), (f, g, r, (H, W, KH, KW, s, d, padding))
    return got


def test_full_grid_matches_the_oracle_field_for_field():
    pads = ['valid', 'same', 0, 1, 2, 5, (0, 0, 0, 0), (1, 2, 3, 4), (3, 0, 0, 2), [2, 1, 0, 0], (0, 5, 1, 0)]
    n = 0
    for H, W, KH, KW, s, d, p in itertools.product([1, 2, 4, 7, 16, 33], [1, 3, 8, 224], [1, 2, 3, 7], [1, 4, 5],
                                                  [1, 2, 3, 5], [1, 2, 3], pads):
        _same(H, W, KH, KW, s, d, p)
        n += 1
    assert n == 6 * 4 * 4 * 3 * 4 * 3 * 11


def test_negative_numerators_truncate_toward_zero_then_clamp():
    """Kernel larger than the padded image: (H + pads - EK) / s + 1 is <= 0 or a fraction in (0, 1); int() of it is 0
    (never -1, which floor division would give for e.g. -3/2 + 1), and max(1, .) makes it 1 (InfoConv2D.py:74-75)."""
    for H, K, s, d in [(2, 7, 1, 1), (2, 7, 2, 1), (2, 7, 3, 1), (1, 5, 2, 3), (3, 4, 5, 2), (1, 8, 7, 1), (4, 3, 2, 4)]:
        for p in ('valid', 0, (0, 0, 0, 0), (0, 0, 1, 0)):
            ci = _same(H, H + 1, K, K, s, d, p)
            assert ci.OH == 1
    # numerator exactly -stride gives 0 -> clamp; numerator -stride+1 .. -1 gives a fraction -> 0 -> clamp
    for s in (1, 2, 3, 4):
        for num in range(-3 * s, 1):
            H, K = 10 + num, 10                       # EK = 10, pads 0: numerator = num
            if H >= 1:
                assert _same(H, H, K, K, s, 1, 0).OH == 1


def test_four_tuples_are_left_top_right_bottom():
    ci = _same(10, 20, 3, 3, 1, 1, (1, 2, 3, 4))
    assert (ci.PADL, ci.PADT, ci.PADR, ci.PADB) == (1, 2, 3, 4)
    assert (ci.OH, ci.OW) == (10 + 2 + 4 - 3 + 1, 20 + 1 + 3 - 3 + 1)
    assert ci.OH_T is None and ci.OW_T is None
    for container in (list, tuple, np.array, lambda t: (x for x in t)):
        got = InfoConv2D(9, 9, 3, 3, 2, 1, container((2, 0, 1, 3)))
        assert (got.PADL, got.PADT, got.PADR, got.PADB, got.OH, got.OW) == (2, 0, 1, 3, 5, 5)


def test_transposed_sizes():
    for H, W, K, s, d in itertools.product([1, 5, 16], [2, 9], [1, 2, 3, 5, 7], [1, 2, 3, 4], [1, 2]):
        v = _same(H, W, K, K, s, d, 'valid')
        sm = _same(H, W, K, K, s, d, 'same')
        assert (sm.OH_T, sm.OW_T) == (H * s, W * s)
        ek = (K - 1) * d + 1
        assert (v.OH_T, v.OW_T) == (H * s + max(ek - s, 0), W * s + max(ek - s, 0))
        # a convolution of the transposed size maps back onto the original size
        back = info_conv2d(v.OH_T, v.OW_T, K, K, s, d, 'valid')
        assert (back.OH, back.OW) == (H, W)
        assert _same(H, W, K, K, s, d, 3).OH_T is None


def test_error_paths_match():
    for bad in ('SAME', 'full', '', None, 1.5, (1, 2), (1, 2, 3), (1, 2, 3, 4, 5), []):
        with pytest.raises(ValueError):
            InfoConv2D(8, 8, 3, 3, 1, 1, bad)
        with pytest.raises(ValueError):
            info_conv2d(8, 8, 3, 3, 1, 1, bad)
    # a bool is an int for isinstance(), there and here (InfoConv2D.py:59)
    assert _same(8, 8, 3, 3, 1, 1, True).PADL == 1
