"""Pins oracle/depthwise.py against the pinned conv2D oracle: a depthwise
convolution is the dense convolution whose kernel is zero off the channel
diagonal."""
import itertools

import numpy as np
import pytest

from oracle import conv2d_all, depthwise_all, depthwise_fwd


def _dense_kernel(k):
    C, KH, KW = k.shape
    w = np.zeros((C, C, KH, KW), k.dtype)
    w[np.arange(C), np.arange(C)] = k
    return w


@pytest.mark.parametrize('padding,s,d,ks', list(itertools.product(['same', 'valid', 1, (2, 0, 1, 3)], [1, 2, 3], [1, 2],
                                                                    [1, 2, 3, 5])))
def test_equals_block_diagonal_dense_convolution(padding, s, d, ks):
    rs = np.random.RandomState(ks * 7 + s)
    x = rs.randint(-4, 5, size=(2, 3, 11, 9)).astype(np.float64)
    k = rs.randint(-4, 5, size=(3, ks, ks + (ks == 2))).astype(np.float64)
    y0 = depthwise_fwd(x, k, s, d, padding)
    dy = rs.randint(-4, 5, size=y0.shape).astype(np.float64)
    y, di, dk = depthwise_all(x, k, dy, s, d, padding)
    ry, rdi, rdw = conv2d_all(x, _dense_kernel(k), dy, s, d, padding)
    assert np.array_equal(y, ry)
    assert np.array_equal(di, rdi)
    assert np.array_equal(dk, rdw[np.arange(3), np.arange(3)])


def test_errors():
    with pytest.raises(ValueError):
        depthwise_fwd(np.zeros((1, 3, 4, 4)), np.zeros((4, 3, 3)))
    with pytest.raises(ValueError):
        depthwise_fwd(np.zeros((1, 3, 4, 4)), np.zeros((3, 1, 3, 3)))
