"""Pins the fp64 conv oracle (conv2D.py:39-54, checker conv2D.py:128-219)
against scipy.signal.correlate2d, an explicit-loop statement of the
definition, special cases that reduce to library routines, and adjoint
identities."""
import itertools

import numpy as np
import pytest
from scipy.signal import correlate2d

from oracle import info_conv2d, conv2d_fwd, conv2d_dx, conv2d_dw, conv2d_all


def _loops(x, w, dy, s, d, padding):
    """Direct statement of the definition: one scalar update per
    (n, o, c, oh, ow, kh, kw) with an in-range test, for Y, dX and dW."""
    N, C, IH, IW = x.shape
    O, _, KH, KW = w.shape
    ci = info_conv2d(IH, IW, KH, KW, s, d, padding)
    y = np.zeros((N, O, ci.OH, ci.OW))
    dx = np.zeros(x.shape)
    dw = np.zeros(w.shape)
    for oh, ow, kh, kw in itertools.product(range(ci.OH), range(ci.OW), range(KH), range(KW)):
        ih = -ci.PADT + kh * d + oh * s
        iw = -ci.PADL + kw * d + ow * s
        if 0 <= ih < IH and 0 <= iw < IW:
            y[:, :, oh, ow] += x[:, :, ih, iw] @ w[:, :, kh, kw].T
            if dy is not None:
                dx[:, :, ih, iw] += dy[:, :, oh, ow] @ w[:, :, kh, kw]
                dw[:, :, kh, kw] += dy[:, :, oh, ow].T @ x[:, :, ih, iw]
    return y, dx, dw


def _cases():
    for padding, d, s, ks in itertools.product(['same', 'valid', 0, 1, 2], [1, 2], [1, 2, 3], [7, 5, 3, 1, 2, 4]):
        for n, ic, oc, hw in [(1, 1, 1, 4), (2, 2, 3, 8), (1, 4, 2, 16)]:
            if padding == 'valid' and hw < ks:
                continue
            yield padding, d, s, ks, n, ic, oc, hw


def test_against_definition_loops_integer_exact():
    rs = np.random.RandomState(0)
    for padding, d, s, ks, n, ic, oc, hw in _cases():
        x = rs.randint(16, size=(n, ic, hw, hw)).astype(np.float64)
        w = rs.randint(16, size=(oc, ic, ks, ks)).astype(np.float64)
        ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
        dy = rs.randint(16, size=(n, oc, ci.OH, ci.OW)).astype(np.float64)
        y, dx, dw = conv2d_all(x, w, dy, s, d, padding)
        ry, rdx, rdw = _loops(x, w, dy, s, d, padding)
        assert y.shape == (n, oc, ci.OH, ci.OW)
        assert np.array_equal(y, ry) and np.array_equal(dx, rdx) and np.array_equal(dw, rdw)


@pytest.mark.parametrize('s,d,ks,pad', [(1, 1, 3, 1), (2, 1, 5, 2), (1, 2, 3, 2), (3, 2, 3, 0), (2, 1, 4, 1)])
def test_forward_against_scipy_correlate(s, d, ks, pad):
    rs = np.random.RandomState(1)
    N, C, O, H, W = 2, 3, 4, 11, 9
    x = rs.uniform(-1, 1, (N, C, H, W))
    w = rs.normal(0, 1, (O, C, ks, ks))
    y = conv2d_fwd(x, w, s, d, pad)
    # dilation -> zero-stuffed kernel; padding -> explicit zero border;
    # stride -> sub-sampling of the stride-1 'valid' correlation
    ek = (ks - 1) * d + 1
    wz = np.zeros((O, C, ek, ek))
    wz[:, :, ::d, ::d] = w
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    ref = np.zeros_like(y)
    for n, o in itertools.product(range(N), range(O)):
        full = sum(correlate2d(xp[n, c], wz[o, c], mode='valid') for c in range(C))
        ref[n, o] = full[::s, ::s][:y.shape[2], :y.shape[3]]
    assert y.shape[2:] == (((H + 2 * pad - ek) // s) + 1, ((W + 2 * pad - ek) // s) + 1)
    np.testing.assert_allclose(y, ref, rtol=0, atol=1e-12)


def test_special_cases_reduce_to_library_routines():
    rs = np.random.RandomState(2)
    x = rs.uniform(-1, 1, (3, 5, 6, 7))
    w = rs.normal(0, 1, (4, 5, 1, 1))
    np.testing.assert_allclose(conv2d_fwd(x, w, 1, 1, 'same'),
                               np.einsum('oc,nchw->nohw', w[:, :, 0, 0], x), atol=1e-12)
    # kernel as large as the image, 'valid' -> one output pixel == matmul
    w = rs.normal(0, 1, (4, 5, 6, 7))
    np.testing.assert_allclose(conv2d_fwd(x, w, 1, 1, 'valid')[:, :, 0, 0],
                               x.reshape(3, -1) @ w.reshape(4, -1).T, atol=1e-12)


def test_adjoint_identities():
    rs = np.random.RandomState(3)
    for padding, d, s, ks, n, ic, oc, hw in _cases():
        x = rs.uniform(-1, 1, (n, ic, hw, hw))
        w = rs.normal(0, 1, (oc, ic, ks, ks))
        y = conv2d_fwd(x, w, s, d, padding)
        dy = rs.normal(0, 1, y.shape)
        dx = conv2d_dx(dy, w, x.shape, s, d, padding)
        dw = conv2d_dw(x, dy, w.shape, s, d, padding)
        lhs = float((y * dy).sum())
        assert abs(lhs - float((x * dx).sum())) <= 1e-9 * max(1.0, abs(lhs))
        assert abs(lhs - float((w * dw).sum())) <= 1e-9 * max(1.0, abs(lhs))


def test_asymmetric_same_padding_even_kernel_and_clamped_output():
    # even kernel + 'same': one more pad on the right/bottom than left/top
    x = np.arange(16, dtype=np.float64).reshape(1, 1, 4, 4)
    w = np.ones((1, 1, 2, 2))
    y = conv2d_fwd(x, w, 1, 1, 'same')
    xp = np.pad(x[0, 0], ((0, 1), (0, 1)))
    np.testing.assert_array_equal(y[0, 0], correlate2d(xp, w[0, 0], mode='valid'))
    # kernel larger than the padded image: output clamped to 1x1
    x = np.ones((1, 1, 4, 4))
    w = np.ones((1, 1, 7, 7))
    y = conv2d_fwd(x, w, 1, 1, 0)
    assert y.shape == (1, 1, 1, 1) and y[0, 0, 0, 0] == 16.0


def test_channel_mismatch_raises():
    with pytest.raises(ValueError):
        conv2d_fwd(np.zeros((1, 3, 4, 4)), np.zeros((2, 4, 3, 3)))
