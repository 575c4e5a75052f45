"""Pins oracle/conv_transpose.py with checks that do not restate its formula."""
import itertools

import numpy as np
import pytest

from oracle import info_conv2d, conv2d_fwd, conv2d_transpose_fwd, conv2d_transpose_di, conv2d_transpose_dk


def _scatter_definition(x, k, s, d, padding):
    """Transposed convolution as the scatter it is defined by: every input
    pixel adds itself times the kernel into the output window it would have
    been computed from by the forward convolution."""
    N, IC, IH, IW = x.shape
    OC, _, KH, KW = k.shape
    ci = info_conv2d(IH, IW, KH, KW, s, d, padding)
    y = np.zeros((N, OC, ci.OH_T, ci.OW_T), np.float64)
    for n, ic, ih, iw, kh, kw in itertools.product(range(N), range(IC), range(IH), range(IW), range(KH), range(KW)):
        oh, ow = ih * s - ci.PADT + kh * d, iw * s - ci.PADL + kw * d
        if 0 <= oh < ci.OH_T and 0 <= ow < ci.OW_T:
            y[n, :, oh, ow] += x[n, ic, ih, iw] * k[:, ic, kh, kw]
    return y


CASES = [(s, d, ks, padding) for padding in ('same', 'valid') for s in (1, 2, 3) for d in (1, 2) for ks in (1, 2, 3, 5)]


@pytest.mark.parametrize('s,d,ks,padding', CASES)
def test_forward_equals_scatter_definition(s, d, ks, padding):
    rs = np.random.RandomState(s * 100 + d * 10 + ks)
    x = rs.randint(8, size=(2, 3, 5, 4)).astype(np.float64)
    k = rs.randint(8, size=(2, 3, ks, ks + (ks == 2))).astype(np.float64)
    assert np.array_equal(conv2d_transpose_fwd(x, k, s, d, padding), _scatter_definition(x, k, s, d, padding))


@pytest.mark.parametrize('s,d,ks,padding', CASES)
def test_adjoint_of_conv2d_and_gradients(s, d, ks, padding):
    """<convT(x, K), z> = <x, conv(z, K^T)> with the pinned conv2D oracle; dI is that conv; dK is the
    gradient of the bilinear form in K (exact on integers)."""
    rs = np.random.RandomState(7 + s * 100 + d * 10 + ks)
    x = rs.randint(-4, 5, size=(2, 3, 6, 5)).astype(np.float64)
    k = rs.randint(-4, 5, size=(4, 3, ks, ks)).astype(np.float64)
    y = conv2d_transpose_fwd(x, k, s, d, padding)
    z = rs.randint(-4, 5, size=y.shape).astype(np.float64)
    kt = np.ascontiguousarray(k.transpose(1, 0, 2, 3))            # (IC, OC, KH, KW): conv2D kernel from z to x
    back = conv2d_fwd(z, kt, s, d, padding)
    assert back.shape == x.shape
    assert np.sum(y * z) == np.sum(x * back)
    assert np.array_equal(conv2d_transpose_di(z, k, x.shape, s, d, padding), back)
    e = rs.randint(-3, 4, size=k.shape).astype(np.float64)
    dk = conv2d_transpose_dk(x, z, k.shape, s, d, padding)
    assert np.sum((conv2d_transpose_fwd(x, k + e, s, d, padding) - y) * z) == np.sum(e * dk)


def test_stride_one_is_convolution_with_flipped_kernel():
    rs = np.random.RandomState(3)
    x = rs.randint(8, size=(1, 2, 7, 6)).astype(np.float64)
    k = rs.randint(8, size=(3, 2, 3, 3)).astype(np.float64)
    y = conv2d_transpose_fwd(x, k, 1, 1, 'same')
    kf = np.ascontiguousarray(k[:, :, ::-1, ::-1])                 # odd kernel, 'same': symmetric pads
    assert np.array_equal(y, conv2d_fwd(x, kf, 1, 1, 'same'))


def test_shapes_and_errors():
    x, k = np.zeros((2, 3, 4, 4)), np.zeros((5, 3, 3, 3))
    assert conv2d_transpose_fwd(x, k, 2, 1, 'same').shape == (2, 5, 8, 8)
    assert conv2d_transpose_fwd(x, k, 2, 1, 'valid').shape == (2, 5, 9, 9)
    assert conv2d_transpose_fwd(x, k, 3, 1, 'valid').shape == (2, 5, 12, 12)
    with pytest.raises(ValueError):
        conv2d_transpose_fwd(x, k, 2, 1, 1)
    with pytest.raises(ValueError):
        conv2d_transpose_fwd(x, np.zeros((5, 4, 3, 3)), 2, 1, 'same')
