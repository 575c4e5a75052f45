"""Pins the integer unfold index maps (unfold2D.py:85-137) by brute-force
nested loops on the reference's own test grid (conv2D.py:77-85) and by the
exact integer adjoint identity between the plain and the transposed map."""
import itertools

import numpy as np
import pytest

from oracle import info_conv2d, unfold_index_map, unfold_T_index_map, apply_index_map


def _grid(small=True):
    for padding, d, s, ks in itertools.product(['same', 'valid', 0, 1, 2], [1, 2], [1, 2, 3], [7, 5, 3, 1]):
        for n, c, hw in [(1, 1, 4), (2, 2, 8), (1, 3, 16)] if small else itertools.product([1, 4], [1, 2, 4], [4, 8, 16]):
            if padding == 'valid' and hw < ks:
                continue
            yield padding, d, s, ks, n, c, hw


def _brute_plain(N, C, H, W, OH, OW, KH, KW, PL, PT, d, s, order):
    out = []
    if order == 'CJI_NHW':
        it = itertools.product(range(C), range(KH), range(KW), range(N), range(OH), range(OW))
        pick = lambda t: (t[3], t[0], t[4], t[5], t[1], t[2])
    else:
        it = itertools.product(range(N), range(OH), range(OW), range(C), range(KH), range(KW))
        pick = lambda t: (t[0], t[3], t[1], t[2], t[4], t[5])
    for t in it:
        n, c, oh, ow, kh, kw = pick(t)
        ih = -PT + kh * d + oh * s
        iw = -PL + kw * d + ow * s
        out.append(((n * C + c) * H + ih) * W + iw if 0 <= ih < H and 0 <= iw < W else -1)
    return np.array(out, np.int64)


def _brute_T(N, O, OH, OW, IH, IW, KH, KW, PL, PT, d, s):
    # order N, H(ih), W(iw), C(o), J(kh), I(kw); source dY[N, O, OH, OW]
    out = []
    for n, ih, iw, o, kh, kw in itertools.product(range(N), range(IH), range(IW), range(O), range(KH), range(KW)):
        hit = -1
        for oh in range(OH):
            if ih == -PT + kh * d + oh * s:
                for ow in range(OW):
                    if iw == -PL + kw * d + ow * s:
                        hit = ((n * O + o) * OH + oh) * OW + ow
        out.append(hit)
    return np.array(out, np.int64)


def test_plain_maps_match_brute_force():
    cnt = 0
    for padding, d, s, ks, n, c, hw in _grid():
        ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
        for order in ('CJI_NHW', 'NHW_CJI'):
            shape, m = unfold_index_map(n, c, hw, hw, ci.OH, ci.OW, ks, ks, ci.PADL, ci.PADT, d, s, order)
            ref = _brute_plain(n, c, hw, hw, ci.OH, ci.OW, ks, ks, ci.PADL, ci.PADT, d, s, order)
            assert m.dtype == np.int64 and np.array_equal(m, ref)
            ckk, p = c * ks * ks, n * ci.OH * ci.OW
            assert shape == ((ckk, p) if order == 'CJI_NHW' else (p, ckk))
        cnt += 1
    assert cnt > 300


def test_transposed_map_matches_brute_force():
    for padding, d, s, ks, n, c, hw in _grid():
        if hw > 8:
            continue
        ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
        o = 2
        shape, m = unfold_T_index_map(n, o, ci.OH, ci.OW, hw, hw, ks, ks, ci.PADL, ci.PADT, d, s)
        ref = _brute_T(n, o, ci.OH, ci.OW, hw, hw, ks, ks, ci.PADL, ci.PADT, d, s)
        assert np.array_equal(m, ref)
        assert shape == (n * hw * hw, o * ks * ks)


def test_transposed_is_exact_adjoint_of_plain():
    """<im2row(X), Z> == <X, col2im(Z)> in exact integer arithmetic, where
    col2im is expressed through the transposed map applied per channel."""
    rs = np.random.RandomState(7)
    for padding, d, s, ks, n, c, hw in _grid():
        ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
        OH, OW = ci.OH, ci.OW
        # plain map with C=1 per (n): rows p=(n,oh,ow), cols (kh,kw)
        shp, mp = unfold_index_map(n, 1, hw, hw, OH, OW, ks, ks, ci.PADL, ci.PADT, d, s, 'NHW_CJI')
        sht, mt = unfold_T_index_map(n, 1, OH, OW, hw, hw, ks, ks, ci.PADL, ci.PADT, d, s, 'NHW_CJI')
        x = rs.randint(0, 16, size=n * hw * hw).astype(np.int64)
        g = rs.randint(0, 16, size=n * OH * OW).astype(np.int64)     # one value per output pixel
        kk = rs.randint(0, 16, size=ks * ks).astype(np.int64)        # one value per tap
        # forward: y[p] = sum_tap im2row(x)[p, tap] * kk[tap]
        y = apply_index_map(x, shp, mp) @ kk
        # adjoint: dx[pix] = sum_tap im2rowT(g)[pix, tap] * kk[tap]
        dx = apply_index_map(g, sht, mt) @ kk
        assert int(y @ g) == int(x @ dx)


def test_pad_right_bottom_do_not_enter_the_map():
    # only PADL/PADT appear in the kernel text; PADR/PADB act through OH/OW
    a = unfold_index_map(1, 1, 8, 8, 8, 8, 4, 4, 1, 1, 1, 1)[1]
    ci = info_conv2d(8, 8, 4, 4, 1, 1, 'same')
    assert (ci.PADL, ci.PADR, ci.OH) == (1, 2, 8)
    b = unfold_index_map(1, 1, 8, 8, ci.OH, ci.OW, 4, 4, ci.PADL, ci.PADT, 1, 1)[1]
    assert np.array_equal(a, b)
