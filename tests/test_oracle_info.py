"""Pins oracle.info_conv2d (restating InfoConv2D.py:41-77) by closed forms,
invariants and the literal shape table of the benchmark configurations."""
import itertools
import math

import pytest

from oracle import info_conv2d


def test_benchmark_config_shapes():
    # (H, W, K, stride, dilation, padding) -> (OH, OW, PADL, PADT)
    table = [
        ((64, 64, 3, 1, 1, 'same'), (64, 64, 1, 1)),       # cfg1
        ((56, 56, 3, 1, 1, 'same'), (56, 56, 1, 1)),       # cfg3
        ((224, 224, 7, 2, 1, 3), (112, 112, 3, 3)),        # cfg4a
        ((28, 28, 1, 1, 1, 'same'), (28, 28, 0, 0)),       # cfg4b
        ((64, 64, 3, 1, 2, 2), (64, 64, 2, 2)),            # cfg4c
        ((128, 128, 5, 2, 1, 2), (64, 64, 2, 2)),          # cfg5 L1
        ((64, 64, 5, 2, 1, 2), (32, 32, 2, 2)),            # cfg5 L2
        ((32, 32, 5, 2, 1, 2), (16, 16, 2, 2)),            # cfg5 L3
        ((16, 16, 5, 2, 1, 2), (8, 8, 2, 2)),              # cfg5 L4
    ]
    for (H, W, K, s, d, p), (OH, OW, PL, PT) in table:
        ci = info_conv2d(H, W, K, K, s, d, p)
        assert (ci.OH, ci.OW, ci.PADL, ci.PADT) == (OH, OW, PL, PT)


@pytest.mark.parametrize('K,d', list(itertools.product(range(1, 9), [1, 2, 3])))
def test_same_padding_invariants(K, d):
    EK = (K - 1) * d + 1
    for H in (4, 7, 16, 33):
        ci = info_conv2d(H, H + 1, K, K, 1, d, 'same')
        assert ci.OH == H and ci.OW == H + 1            # stride 1 keeps the size
        assert ci.PADL + ci.PADR == EK - 1 and ci.PADT + ci.PADB == EK - 1
        if EK % 2 == 1:
            assert ci.PADL == ci.PADR
        else:
            assert ci.PADR == ci.PADL + 1 and ci.PADB == ci.PADT + 1
        for s in (2, 3):
            cs = info_conv2d(H, H, K, K, s, d, 'same')
            assert cs.OH == (H - 1) // s + 1            # ceil(H / s)
            assert (cs.OH_T, cs.OW_T) == (H * s, H * s)


def test_textbook_formula_and_clamp():
    for H, K, s, d, p in itertools.product([1, 4, 8, 16, 31], [1, 3, 5, 7], [1, 2, 3], [1, 2], [0, 1, 2, 5]):
        EK = (K - 1) * d + 1
        ci = info_conv2d(H, H, K, K, s, d, p)
        num = H + 2 * p - EK
        if num >= 0:
            assert ci.OH == num // s + 1
        else:
            # float quotient + 1 truncated toward zero, then clamped to >= 1
            assert ci.OH == max(1, math.trunc(num / s + 1))
        assert ci.OH >= 1 and ci.OW >= 1
        assert ci.OH_T is None


def test_valid_and_tuple_and_errors():
    ci = info_conv2d(8, 10, 3, 5, 2, 1, 'valid')
    assert (ci.PADL, ci.PADT, ci.PADR, ci.PADB) == (0, 0, 0, 0)
    assert (ci.OH, ci.OW) == (3, 3)
    assert (ci.OH_T, ci.OW_T) == (8 * 2 + 1, 10 * 2 + 3)
    ci = info_conv2d(8, 8, 3, 3, 1, 1, (1, 2, 3, 4))
    assert (ci.PADL, ci.PADT, ci.PADR, ci.PADB) == (1, 2, 3, 4)
    assert (ci.OH, ci.OW) == (8 + 2 + 4 - 3 + 1, 8 + 1 + 3 - 3 + 1)
    with pytest.raises(ValueError):
        info_conv2d(8, 8, 3, 3, 1, 1, (1, 2, 3))
    with pytest.raises(ValueError):
        info_conv2d(8, 8, 3, 3, 1, 1, 1.5)
    with pytest.raises(ValueError):
        info_conv2d(8, 8, 3, 3, 1, 1, 'full')
