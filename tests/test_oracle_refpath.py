"""The fp32 C restatement of the reference data flow (unfold -> register
tiled GeMM -> transpose, matmul.py:106-164) must agree with the fp64 oracle:
exactly on small-integer data, to 1e-5 on random data; its unfold must equal
the integer index maps bit for bit."""
import itertools

import numpy as np
import pytest

from oracle import (info_conv2d, conv2d_all, unfold_index_map, unfold_T_index_map,
                    apply_index_map, matmul_fwd, matmul_da, matmul_db)
from oracle import refpath


def test_tile_width_rule():
    # matmul.py:106-113
    assert refpath.gemm_tile_widths(100352, 128, 1152) == (16, 8)    # cfg3 fwd
    assert refpath.gemm_tile_widths(32768, 32, 27) == (16, 1)        # cfg1 fwd
    assert refpath.gemm_tile_widths(3, 12, 8) == (1, 4)
    assert refpath.gemm_tile_widths(6, 7, 7) == (2, 1)


def test_unfold_matches_index_maps_bit_exact():
    for padding, d, s, ks in itertools.product(['same', 'valid', 1], [1, 2], [1, 2, 3], [5, 3, 2, 1]):
        n, c, hw, o = 2, 3, 8, 2
        ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
        x = np.arange(1, n * c * hw * hw + 1, dtype=np.float32)      # value = flat index + 1
        for order, name in ((0, 'CJI_NHW'), (1, 'NHW_CJI')):
            got = refpath.unfold2d(x, n, c, hw, hw, ci.OH, ci.OW, ks, ks, ci.PADL, ci.PADT, d, s, order, False)
            _, m = unfold_index_map(n, c, hw, hw, ci.OH, ci.OW, ks, ks, ci.PADL, ci.PADT, d, s, name)
            assert np.array_equal(got.astype(np.int64) - 1, m)
        dy = np.arange(1, n * o * ci.OH * ci.OW + 1, dtype=np.float32)
        got = refpath.unfold2d(dy, n, o, ci.OH, ci.OW, hw, hw, ks, ks, ci.PADL, ci.PADT, d, s, 1, True)
        _, m = unfold_T_index_map(n, o, ci.OH, ci.OW, hw, hw, ks, ks, ci.PADL, ci.PADT, d, s)
        assert np.array_equal(got.astype(np.int64) - 1, m)


def test_conv_integer_exact_with_accumulate():
    rs = np.random.RandomState(0)
    for padding, d, s, ks in itertools.product(['same', 'valid', 0, 2], [1, 2], [1, 2, 3], [7, 3, 1]):
        for n, ic, oc, hw in [(1, 1, 1, 8), (4, 2, 4, 8), (1, 4, 2, 16)]:
            if padding == 'valid' and hw < ks:
                continue
            x = rs.randint(16, size=(n, ic, hw, hw)).astype(np.float32)
            w = rs.randint(16, size=(oc, ic, ks, ks)).astype(np.float32)
            ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
            dy = rs.randint(16, size=(n, oc, ci.OH, ci.OW)).astype(np.float32)
            y, dx, dw = conv2d_all(x, w, dy, s, d, padding)
            assert np.array_equal(refpath.conv2d_fwd(x, w, s, d, padding), y)
            gx = np.ones(x.shape, np.float32)
            gw = np.ones(w.shape, np.float32)
            refpath.conv2d_dx(dy, w, x.shape, s, d, padding, into=gx)
            refpath.conv2d_dw(x, dy, w.shape, s, d, padding, into=gw)
            assert np.array_equal(gx - 1.0, dx) and np.array_equal(gw - 1.0, dw)


def test_conv_random_fp32_close_to_fp64():
    rs = np.random.RandomState(1)
    x = rs.uniform(-1, 1, (4, 16, 20, 20)).astype(np.float32)
    w = rs.normal(0, np.sqrt(2 / (16 * 9)), (24, 16, 3, 3)).astype(np.float32)
    dy = rs.normal(0, 1, (4, 24, 20, 20)).astype(np.float32)
    y, dx, dw = conv2d_all(x, w, dy)
    for got, ref in ((refpath.conv2d_fwd(x, w), y), (refpath.conv2d_dx(dy, w, x.shape), dx),
                     (refpath.conv2d_dw(x, dy, w.shape), dw)):
        assert np.abs(got - ref).max() / np.abs(ref).max() <= 1e-5


def test_matmul_integer_exact_and_transpose():
    rs = np.random.RandomState(2)
    for batch, M, K, N in [(1, 1, 1, 1), (1, 5, 7, 3), (3, 8, 32, 16), (2, 6, 12, 20), (1, 16, 64, 48)]:
        ash, bsh = ((M, K), (K, N)) if batch == 1 else ((batch, M, K), (batch, K, N))
        a = rs.randint(16, size=ash).astype(np.float32)
        b = rs.randint(16, size=bsh).astype(np.float32)
        assert np.array_equal(refpath.matmul(a, b), matmul_fwd(a, b))
        dc = rs.randint(8, size=b.shape[:-2] + (M, N)).astype(np.float32)
        da, db = refpath.matmul_bwd(a, b, dc, np.ones(ash, np.float32), np.ones(bsh, np.float32))
        assert np.array_equal(da - 1, matmul_da(dc, b, a.shape))
        assert np.array_equal(db - 1, matmul_db(a, dc, b.shape))
    t = rs.randint(256, size=(3, 4, 5, 6)).astype(np.float32)
    assert np.array_equal(refpath.transpose(t, (2, 0, 3, 1)), t.transpose(2, 0, 3, 1))
