"""GPU parity tests of the C ABI (liblitenn_hip.so) against the CPU oracle.

Bars: bit-exact on integer-valued data (the reference's own test trick,
conv2D.py:90-115, matmul.py:192-225: all partial sums are exactly
representable, so the result does not depend on summation order) and
normalised max error <= 1e-4 against the fp64 oracle on the seeded float
data of the benchmark configurations.
"""
import itertools

import numpy as np
import pytest

from oracle import depthwise_all, hash_rng
from oracle import (info_conv2d, conv2d_all, conv2d_fwd, conv2d_dx, conv2d_dw, unfold_index_map,
                    unfold_T_index_map, matmul_fwd)
from tests.gpu_util import DevArr, rel_err, say

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _desc(api, xs, ws, s, d, padding):
    N, C, IH, IW = xs
    O, _, KH, KW = ws
    ci = info_conv2d(IH, IW, KH, KW, s, d, padding)
    return api.conv_desc(N, C, IH, IW, O, KH, KW, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d), ci


def _run_conv(api, x, w, dy, s, d, padding, prefill=None):
    """fwd (beta 0), dgrad and wgrad through the C ABI.  prefill=None: grads
    written with beta 0; else grads pre-filled with that value and beta 1."""
    desc, ci = _desc(api, x.shape, w.shape, s, d, padding)
    X, W, dY = DevArr(api, x), DevArr(api, w), DevArr(api, dy)
    Y = DevArr(api, shape=dy.shape, fill=np.nan)
    beta = 0 if prefill is None else 1
    dX = DevArr(api, shape=x.shape, fill=np.nan if prefill is None else prefill)
    dW = DevArr(api, shape=w.shape, fill=np.nan if prefill is None else prefill)
    api.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, 0)
    api.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
    api.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, beta)
    return Y.get(), dX.get(), dW.get()


# ------------------------------------------------------------------ GEMM
@pytest.mark.parametrize('ta,tb', [(0, 0), (0, 1), (1, 0)])
def test_gemm_integer_exact(hip, ta, tb):
    rs = np.random.RandomState(10 + 2 * ta + tb)
    shapes = [(1, 1, 1, 1), (1, 5, 7, 3), (1, 33, 65, 17), (1, 128, 128, 16), (1, 130, 257, 100),
              (3, 8, 32, 16), (2, 70, 40, 24), (1, 64, 512, 48), (1, 256, 384, 160), (1, 2, 3000, 5),
              (4, 1, 9, 1), (1, 97, 31, 1000),
              # 16-byte aligned rows and K a multiple of 32: operands go straight into LDS
              (1, 128, 256, 64), (2, 36, 100, 32), (1, 20, 44, 96), (3, 132, 260, 128), (1, 68, 8, 32),
              (1, 4, 4, 32), (1, 516, 96, 64), (1, 64, 1028, 320)]
    for batch, M, N, K in shapes:
        say(f'gemm ta={ta} tb={tb} batch={batch} M={M} N={N} K={K}')
        a = rs.randint(16, size=(batch, K, M) if ta else (batch, M, K)).astype(np.float32)
        b = rs.randint(16, size=(batch, N, K) if tb else (batch, K, N)).astype(np.float32)
        c0 = rs.randint(8, size=(batch, M, N)).astype(np.float32)
        ref = np.matmul(a.transpose(0, 2, 1) if ta else a, b.transpose(0, 2, 1) if tb else b)
        A, B = DevArr(hip, a), DevArr(hip, b)
        for beta in (0, 1):
            C = DevArr(hip, c0)
            hip.gemm(0, ta, tb, batch, M, N, K, A.ptr, a.shape[2], a.shape[1] * a.shape[2],
                     B.ptr, b.shape[2], b.shape[1] * b.shape[2], C.ptr, N, M * N, beta)
            got = C.get()
            assert np.array_equal(got, ref + (c0 if beta else 0)), (batch, M, N, K, beta)


def test_gemm_leading_dimensions_and_unaligned(hip):
    rs = np.random.RandomState(3)
    M, N, K, lda, ldb, ldc = 45, 70, 37, 41, 75, 77
    a = rs.randint(16, size=(M, lda)).astype(np.float32)
    b = rs.randint(16, size=(K, ldb)).astype(np.float32)
    c0 = rs.randint(16, size=(M, ldc)).astype(np.float32)
    A, B, C = DevArr(hip, a), DevArr(hip, b), DevArr(hip, c0)
    say('gemm with padded leading dimensions')
    hip.gemm(0, 0, 0, 1, M, N, K, A.ptr, lda, 0, B.ptr, ldb, 0, C.ptr, ldc, 0, 0)
    got = C.get()
    assert np.array_equal(got[:, :N], a[:, :K] @ b[:, :N])
    assert np.array_equal(got[:, N:], c0[:, N:])          # padding columns untouched
    # operands that start 4 bytes into an allocation take the scalar-load path
    a2 = rs.randint(16, size=(64 * 64 + 1)).astype(np.float32)
    A2 = DevArr(hip, a2)
    b2 = rs.randint(16, size=(64, 64)).astype(np.float32)
    B2, C2 = DevArr(hip, b2), DevArr(hip, shape=(64, 64), fill=0.0)
    say('gemm with a 4-byte-offset operand')
    hip.gemm(0, 0, 0, 1, 64, 64, 64, A2.ptr + 4, 64, 0, B2.ptr, 64, 0, C2.ptr, 64, 0, 0)
    assert np.array_equal(C2.get(), a2[1:].reshape(64, 64) @ b2)


def test_gemm_float_tolerance(hip):
    rs = np.random.RandomState(0)
    M = N = K = 768
    a, b, dc = (rs.normal(0, 1, (M, K)).astype(np.float32) for _ in range(3))
    A, B, D = DevArr(hip, a), DevArr(hip, b), DevArr(hip, dc)
    C, dA, dB = (DevArr(hip, shape=(M, N), fill=0.0) for _ in range(3))
    say('gemm 768^3 fwd / dA / dB')
    hip.gemm(0, 0, 0, 1, M, N, K, A.ptr, K, 0, B.ptr, N, 0, C.ptr, N, 0, 0)
    hip.gemm(0, 0, 1, 1, M, K, N, D.ptr, N, 0, B.ptr, N, 0, dA.ptr, K, 0, 1)
    hip.gemm(0, 1, 0, 1, K, N, M, A.ptr, K, 0, D.ptr, N, 0, dB.ptr, N, 0, 1)
    a64, b64, d64 = a.astype(np.float64), b.astype(np.float64), dc.astype(np.float64)
    assert rel_err(C.get(), a64 @ b64) <= TOL
    assert rel_err(dA.get(), d64 @ b64.T) <= TOL
    assert rel_err(dB.get(), a64.T @ d64) <= TOL


def test_gemm_argument_errors(hip):
    A = DevArr(hip, shape=(16, 16), fill=0.0)
    with pytest.raises(hip.HipException) as e:
        hip.gemm(0, 0, 0, 1, 16, 16, 0, A.ptr, 16, 0, A.ptr, 16, 0, A.ptr, 16, 0, 0)
    assert e.value.code == hip.ERR_INVALID
    with pytest.raises(hip.HipException):
        hip.gemm(0, 0, 0, 1, 16, 16, 16, A.ptr, 8, 0, A.ptr, 16, 0, A.ptr, 16, 0, 0)
    with pytest.raises(hip.HipException) as e:
        hip.gemm(0, 1, 1, 1, 16, 16, 16, A.ptr, 16, 0, A.ptr, 16, 0, A.ptr, 16, 0, 0)
    assert e.value.code == hip.ERR_UNSUPPORTED
    with pytest.raises(hip.HipException) as e:
        hip.malloc(99, 16)
    assert e.value.code == hip.ERR_NO_DEVICE


# ------------------------------------------------------------------ conv
def _grid(pads):
    # the reference's own grid (conv2D.py:77-85)
    for padding, d, s, ks, n, ic, oc, hw in itertools.product(pads, [1, 2], [1, 2, 3], [7, 5, 3, 1], [1, 4],
                                                                [1, 2, 4], [1, 2, 4], [4, 8, 16]):
        if padding == 'valid' and hw < ks:
            continue
        yield padding, d, s, ks, n, ic, oc, hw


@pytest.mark.parametrize('pads', [['same'], ['valid'], [0], [1], [2]])
def test_conv_reference_grid_integer_exact(hip, pads):
    """Every case of the reference's conv2d_test: Y exact; gradients written
    into buffers pre-filled with 1.0 must equal 1 + oracle (pins '+=')."""
    rs = np.random.RandomState(len(str(pads)) * 7 + (pads[0] if isinstance(pads[0], int) else 0))
    cnt = 0
    for padding, d, s, ks, n, ic, oc, hw in _grid(pads):
        if cnt % 100 == 0:
            say(f'conv grid padding={padding} case {cnt}: d={d} s={s} ks={ks} n={n} ic={ic} oc={oc} hw={hw}')
        x = rs.randint(16, size=(n, ic, hw, hw)).astype(np.float32)
        w = rs.randint(16, size=(oc, ic, ks, ks)).astype(np.float32)
        ci = info_conv2d(hw, hw, ks, ks, s, d, padding)
        dy = rs.randint(16, size=(n, oc, ci.OH, ci.OW)).astype(np.float32)
        y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding, prefill=1.0)
        ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
        tag = (padding, d, s, ks, n, ic, oc, hw)
        assert np.array_equal(y, ry), ('fwd', tag)
        assert np.array_equal(dx - 1.0, rdx), ('dX', tag)
        assert np.array_equal(dw - 1.0, rdw), ('dW', tag)
        cnt += 1
    assert cnt > 500


def test_conv_odd_corners_integer_exact(hip):
    """Even kernels with asymmetric 'same' padding, non-square images and
    kernels, explicit 4-tuple pads, output clamped to 1x1, many channels
    (several M tiles, ragged K), large strides."""
    rs = np.random.RandomState(5)
    cases = [
        ((2, 3, 9, 7), (5, 3, 2, 4), 1, 1, 'same'), ((1, 2, 4, 4), (3, 2, 7, 7), 1, 1, 0),
        ((2, 5, 12, 10), (6, 5, 3, 2), 2, 1, (1, 2, 0, 3)), ((1, 130, 6, 6), (70, 130, 3, 3), 1, 1, 'same'),
        ((3, 33, 10, 10), (129, 33, 1, 1), 1, 1, 'same'), ((2, 4, 20, 20), (4, 4, 3, 3), 4, 3, 2),
        ((1, 1, 40, 40), (1, 1, 5, 5), 3, 2, 'same'), ((2, 16, 17, 13), (40, 16, 4, 4), 2, 1, 'same'),
        ((1, 7, 30, 30), (9, 7, 3, 3), 1, 1, 'valid'), ((5, 3, 8, 8), (2, 3, 8, 8), 1, 1, 'valid'),
    ]
    for xs, ws, s, d, padding in cases:
        say(f'conv corner x={xs} w={ws} s={s} d={d} pad={padding}')
        x = rs.randint(8, size=xs).astype(np.float32)
        w = rs.randint(8, size=ws).astype(np.float32)
        ci = info_conv2d(xs[2], xs[3], ws[2], ws[3], s, d, padding)
        dy = rs.randint(8, size=(xs[0], ws[0], ci.OH, ci.OW)).astype(np.float32)
        ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
        for prefill in (None, 2.0):
            y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding, prefill=prefill)
            off = 0.0 if prefill is None else prefill
            assert np.array_equal(y, ry), ('fwd', xs, ws)
            assert np.array_equal(dx - off, rdx), ('dX', xs, ws)
            assert np.array_equal(dw - off, rdw), ('dW', xs, ws)


def test_conv_strided_dgrad_pixel_classes_integer_exact(hip):
    """dX of a strided convolution is computed per class of input pixels
    ((ih + PADT) mod S, (iw + PADL) mod S).  Sweep strides against dilations
    and kernel sizes so that classes with no tap, with no pixel, with one tap
    and with uneven tap counts all occur, on the table-driven path (odd
    channel counts) and on the tap-major path (O a multiple of 32), with and
    without accumulation into a prefilled dX."""
    rs = np.random.RandomState(11)
    cnt = 0
    for s in (2, 3, 4):
        for d in (1, 2, 3):
            for k in (1, 2, 3, 5):
                for padding in ('same', 'valid', 1, (2, 0, 1, 3)):
                    for (C, O) in ((3, 5), (6, 32), (33, 64)):
                        H, W_ = 11 + s, 9 + 2 * s
                        try:
                            ci = info_conv2d(H, W_, k, k + (s == 3), s, d, padding)
                        except ValueError:
                            continue
                        if ci.OH <= 0 or ci.OW <= 0:
                            continue
                        xs, ws = (2, C, H, W_), (O, C, k, k + (s == 3))
                        say(f'conv classes x={xs} w={ws} s={s} d={d} pad={padding}')
                        x = rs.randint(5, size=xs).astype(np.float32)
                        w = rs.randint(5, size=ws).astype(np.float32)
                        dy = rs.randint(5, size=(xs[0], O, ci.OH, ci.OW)).astype(np.float32)
                        ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
                        prefill = None if cnt % 2 else 3.0
                        y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding, prefill=prefill)
                        off = 0.0 if prefill is None else prefill
                        assert np.array_equal(y, ry), ('fwd', xs, ws, s, d, padding)
                        assert np.array_equal(dx - off, rdx), ('dX', xs, ws, s, d, padding)
                        assert np.array_equal(dw - off, rdw), ('dW', xs, ws, s, d, padding)
                        cnt += 1
    assert cnt > 300


def test_conv_strided_dgrad_paired_classes_integer_exact(hip):
    """Stride 2 with 33-64 input channels (a multiple of 4) and class planes of at least 512 sub-tiles of 64 x 128 each:
    the four pixel classes run on 64 x 128 tiles, two workgroups per compute unit, ordered so that a class with many
    taps shares its compute units with one with few.  Whole and ragged tiles, 5x5 and 3x3, '=' and '+='; the data
    gradient through lnn_conv2d_dgrad_f32 and, on one permuted copy, lnn_conv2d_dgrad_pw_f32.  The first image is
    checked against the oracle, all images against the same call on half the batch at a time (class planes too small
    for this plan: the wider tiles, one workgroup per compute unit, which the other tests pin).  Exact on small
    integers."""
    rs = np.random.RandomState(66)
    for xs, ws, padding in [((16, 64, 64, 64), (32, 64, 5, 5), 2), ((17, 48, 62, 66), (32, 48, 3, 3), 'same'),
                            ((9, 36, 91, 90), (64, 36, 5, 5), (1, 2, 2, 1))]:
        desc, ci = _desc(hip, xs, ws, 2, 1, padding)
        say(f'paired classes x={xs} w={ws} pad={padding}')
        n, O = xs[0], ws[0]
        w = rs.randint(-2, 3, size=ws).astype(np.float32)
        dy = rs.randint(-2, 3, size=(n, O, ci.OH, ci.OW)).astype(np.float32)
        W, dY = DevArr(hip, w), DevArr(hip, dy)
        ref = np.empty(xs, np.float32)
        half = (n + 1) // 2
        for i0 in range(0, n, half):
            m = min(half, n - i0)
            dpart, _ = _desc(hip, (m,) + xs[1:], ws, 2, 1, padding)
            dYp, dXp = DevArr(hip, dy[i0:i0 + m]), DevArr(hip, shape=(m,) + xs[1:], fill=np.nan)
            hip.conv2d_dgrad(0, dpart, dYp.ptr, W.ptr, dXp.ptr, 0)
            ref[i0:i0 + m] = dXp.get()
        assert np.array_equal(ref[:1], conv2d_dx(dy[:1], w, (1,) + xs[1:], 2, 1, padding)), (xs, ws, padding)
        Wp = DevArr(hip, shape=(O, ws[2] * ws[3], ws[1]), fill=np.nan)
        hip.conv2d_permute_weights(0, desc, W.ptr, hip.W_OIHW, Wp.ptr)
        for beta, fill in ((0, np.nan), (1, -1.0)):
            dX = DevArr(hip, shape=xs, fill=fill)
            hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
            assert np.array_equal(dX.get() - (-1.0 if beta else 0.0), ref), (xs, ws, padding, beta)
            dX = DevArr(hip, shape=xs, fill=fill)
            hip.conv2d_dgrad_pw(0, desc, dY.ptr, Wp.ptr, dX.ptr, beta)
            assert np.array_equal(dX.get() - (-1.0 if beta else 0.0), ref), (xs, ws, padding, beta, 'pw')


def test_conv_channel_multiples_of_32_integer_exact(hip):
    """Channel counts that are multiples of 32 take the tap-major kernels
    (forward / dgrad: permuted weights, address arithmetic in the scalar
    offset; wgrad: pixel-major loaders with tap-major columns, for every tile
    shape the output-channel count selects); everything else about the
    geometry varies, and some pairs stay on the generic kernels."""
    rs = np.random.RandomState(11)
    cnt = 0
    for (ic, oc), s, d, ks, padding in itertools.product([(16, 16), (32, 48), (48, 16), (16, 5), (6, 32), (32, 96),
                                                          (64, 40), (128, 8), (64, 130), (96, 70), (160, 66)],
                                                         [1, 2, 3], [1, 2], [1, 2, 3, 5], ['same', 'valid', 1]):
        n, h, w_ = 2, 11, 9
        if padding == 'valid' and min(h, w_) < (ks - 1) * d + 1:
            continue
        if cnt % 40 == 0:
            say(f'conv c16 case {cnt}: ic={ic} oc={oc} s={s} d={d} ks={ks} pad={padding}')
        x = rs.randint(8, size=(n, ic, h, w_)).astype(np.float32)
        w = rs.randint(8, size=(oc, ic, ks, ks)).astype(np.float32)
        ci = info_conv2d(h, w_, ks, ks, s, d, padding)
        dy = rs.randint(8, size=(n, oc, ci.OH, ci.OW)).astype(np.float32)
        y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding, prefill=1.0)
        ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
        tag = (ic, oc, s, d, ks, padding)
        assert np.array_equal(y, ry), ('fwd', tag)
        assert np.array_equal(dx - 1.0, rdx), ('dX', tag)
        assert np.array_equal(dw - 1.0, rdw), ('dW', tag)
        cnt += 1
    assert cnt > 600


def test_conv_wide_images_pixel_walk_integer_exact(hip):
    """The pixel-major wgrad loaders carry each lane's pixel forward by 32
    per K step with additions and wrap tests: images wider than, equal to and
    narrower than a K step, rows that wrap in the middle of a step, several
    images per K slice, output planes whose size is and is not a multiple of 4."""
    rs = np.random.RandomState(21)
    shapes = [(2, 32, 9, 40), (3, 32, 40, 37), (1, 64, 64, 64), (2, 32, 5, 33), (5, 32, 6, 32), (2, 64, 33, 8),
              (7, 32, 7, 7), (1, 32, 2, 100), (4, 96, 12, 12)]
    for xs in shapes:
        for s, d, ks, padding in ((1, 1, 3, 'same'), (2, 1, 3, 1), (1, 2, 2, 'valid'), (1, 1, 1, 'same'), (2, 1, 5, 2)):
            for oc in (32, 40, 130):
                try:
                    ci = info_conv2d(xs[2], xs[3], ks, ks, s, d, padding)
                except ValueError:
                    continue
                if ci.OH <= 0 or ci.OW <= 0:
                    continue
                say(f'conv walk x={xs} oc={oc} s={s} d={d} ks={ks} pad={padding}')
                x = rs.randint(6, size=xs).astype(np.float32)
                w = rs.randint(6, size=(oc, xs[1], ks, ks)).astype(np.float32)
                dy = rs.randint(6, size=(xs[0], oc, ci.OH, ci.OW)).astype(np.float32)
                ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
                y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding, prefill=None)
                assert np.array_equal(y, ry), ('fwd', xs, oc, s, d, ks, padding)
                assert np.array_equal(dx, rdx), ('dX', xs, oc, s, d, ks, padding)
                assert np.array_equal(dw, rdw), ('dW', xs, oc, s, d, ks, padding)


def test_conv_wgrad_128bit_pixel_gather_integer_exact(hip):
    """Stride 1, an output width that is a multiple of 4 and no padded columns (1x1 kernels, 'valid' convolutions,
    padding at the top / bottom only) send the wgrad pixel gather as 128-bit transfers of four consecutive input
    pixels at any 4-byte alignment; rows above / below the image arrive as zeros.  The same geometries with padded
    columns take the 32-bit gather and are checked beside them."""
    rs = np.random.RandomState(31)
    cases = [((2, 32, 12, 12), 3, 1, 'same'), ((1, 32, 58, 58), 3, 1, 'valid'), ((2, 64, 9, 16), 5, 1, 'same'),
             ((2, 32, 10, 20), 3, 2, 'same'), ((1, 32, 7, 10), 3, 1, 2), ((2, 32, 6, 6), 3, 1, 4),
             ((3, 32, 5, 14), 2, 1, (2, 0, 1, 1)), ((1, 96, 8, 9), 3, 1, (3, 1, 2, 0)), ((2, 32, 6, 8), 7, 1, 'same'),
             ((1, 32, 20, 44), 3, 3, 'same'), ((4, 32, 8, 8), 1, 1, 'same'), ((1, 32, 9, 4), 3, 1, 'same'),
             ((2, 128, 28, 28), 3, 1, 'same'), ((1, 32, 33, 36), 4, 1, (1, 1, 2, 2)),
             ((2, 32, 8, 18), 3, 1, (0, 1, 0, 1)), ((1, 64, 10, 12), 1, 1, (0, 2, 0, 2)), ((2, 32, 9, 20), 3, 2, 'valid'),
             ((3, 32, 6, 11), 4, 1, (0, 3, 0, 3)), ((2, 256, 28, 28), 1, 1, 'same'), ((1, 32, 40, 35), 4, 1, 'valid')]
    for xs, ks, d, padding in cases:
        ci = info_conv2d(xs[2], xs[3], ks, ks, 1, d, padding)
        assert ci.OW % 4 == 0, (xs, ks, d, padding, ci.OW)
        for oc in (32, 72, 130):
            say(f'wgrad gather x={xs} oc={oc} ks={ks} d={d} pad={padding}')
            x = rs.randint(-5, 6, size=xs).astype(np.float32)
            w = rs.randint(-5, 6, size=(oc, xs[1], ks, ks)).astype(np.float32)
            dy = rs.randint(-5, 6, size=(xs[0], oc, ci.OH, ci.OW)).astype(np.float32)
            rdw = conv2d_dw(x, dy, w.shape, 1, d, padding)
            desc, _ = _desc(hip, xs, w.shape, 1, d, padding)
            X, dY = DevArr(hip, x), DevArr(hip, dy)
            for beta, fill in ((0, np.nan), (1, 3.0)):
                dW = DevArr(hip, shape=w.shape, fill=fill)
                hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, beta)
                assert np.array_equal(dW.get() - (3.0 if beta else 0.0), rdw), (xs, oc, ks, d, padding, beta)


def test_conv_dgrad_few_input_channels_vector_kernel_integer_exact(hip):
    """C <= 4, dilation 1, stride 1 (K = 1, 3, 5) or 2 (K = 3, 4, 5, 7) with enough tiles for the chip takes the
    vector-ALU data gradient (all pixel classes of a 16 x 16 tile in one block, a quarter of the output channels per
    wavefront).  Image sizes that are not multiples
    of the tile, every padding kind, '=' and '+=', and the neighbouring shapes that stay on the MFMA path."""
    rs = np.random.RandomState(41)
    vec = [(16, 3, 1, 3, 'same', 5), (16, 4, 1, 5, 'valid', 3), (16, 1, 1, 1, 'same', 6), (16, 2, 1, 3, 2, 4),
           (16, 3, 1, 5, (1, 0, 3, 2), 3), (40, 3, 2, 7, 3, 1), (40, 3, 2, 5, 'same', 3), (40, 4, 2, 4, 1, 3),
           (40, 1, 2, 3, 'valid', 4), (40, 2, 2, 5, (0, 2, 1, 0), 3), (40, 3, 2, 3, 0, 5), (40, 3, 2, 4, (2, 1, 0, 3), 2),
           # each wavefront walks its quarter of the output channels in chunks of 4 held in LDS: wavefronts without
           # channels, ragged last chunks, ragged last quarters, four full chunks each
           (40, 3, 2, 7, 3, 8), (40, 3, 2, 7, 3, 9), (40, 3, 2, 7, 3, 20), (40, 3, 2, 7, 3, 64),
           (16, 3, 1, 3, 'same', 9), (16, 4, 1, 5, 'same', 20), (16, 3, 1, 3, 'same', 64), (16, 1, 1, 5, 2, 8),
           (40, 4, 2, 4, 1, 17), (40, 3, 2, 5, 'same', 64), (40, 2, 2, 3, 1, 16), (16, 3, 1, 1, 0, 33)]
    mfma = [# fewer images, i.e. fewer tiles than compute units: these stay on the MFMA path
            (16, 3, 2, 5, 'same', 3), (16, 4, 2, 7, 3, 2), (6, 3, 1, 3, 'same', 4), (6, 2, 1, 5, (2, 0, 1, 3), 3),
            (16, 1, 2, 4, 1, 3), (16, 3, 2, 3, (1, 0, 0, 1), 4), (16, 3, 2, 7, 3, 20),
            # not covered by the kernel: dilation, stride 3, 7 x 7 at stride 1
            (16, 3, 1, 3, 'same', 4, 2), (30, 3, 3, 5, 2, 3), (16, 3, 1, 7, 'same', 2)]
    cus = hip.device_info(0)['compute_units']
    for case in vec + mfma:
        n, c, s_, k, padding, oc = case[:6]
        d = case[6] if len(case) > 6 else 1
        xs = (n, c, 70, 66)
        ci = info_conv2d(70, 66, k, k, s_, d, padding)
        say(f'small-C dgrad x={xs} oc={oc} k={k} s={s_} d={d} pad={padding}')
        w = rs.randint(-4, 5, size=(oc, c, k, k)).astype(np.float32)
        dy = rs.randint(-4, 5, size=(n, oc, ci.OH, ci.OW)).astype(np.float32)
        ref = conv2d_dx(dy, w, xs, s_, d, padding)
        desc, _ = _desc(hip, xs, w.shape, s_, d, padding)
        W, dY = DevArr(hip, w), DevArr(hip, dy)
        for beta, fill in ((0, np.nan), (1, -2.0)):
            if cus == 256:   # the case lists are laid out for the MI355X's 256 compute units
                path, _ = hip.conv2d_dgrad_path(desc, beta, cus)
                assert (path == hip.DGRAD_PATH_VECTOR) == (case in vec), (case, beta, path)
            dX = DevArr(hip, shape=xs, fill=fill)
            hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
            assert np.array_equal(dX.get() - (-2.0 if beta else 0.0), ref), (case, beta)


def test_conv_dgrad_on_forward_permuted_weights_integer_exact(hip):
    """With O a multiple of 32 and C a multiple of 4 (C > 4) the data gradient reads the weights in the forward
    pass's layout Wp[o][tap][c], whatever the stride and the pixel class: channel counts that give one ragged,
    one full and several row tiles of every tile shape, strides 1-3, dilation, every padding kind, '=' and '+=',
    through lnn_conv2d_dgrad_f32 (copy made in scratch) and through lnn_conv2d_dgrad_pw_f32 on a copy made once
    by lnn_conv2d_permute_weights_f32; the forward pass on the same copy where it reads one."""
    rs = np.random.RandomState(61)
    cnt = 0
    for (C, O), s, d, ks, padding in itertools.product([(8, 32), (12, 64), (20, 32), (36, 96), (64, 64), (132, 32), (32, 160)],
                                                       [1, 2, 3], [1, 2], [1, 2, 3, 5], ['same', 'valid', 1, (2, 0, 1, 3)]):
        n, h, w_ = 2, 11 + s, 9 + 2 * s
        try:
            ci = info_conv2d(h, w_, ks, ks, s, d, padding)
        except ValueError:
            continue
        if padding == 'valid' and min(h, w_) < (ks - 1) * d + 1:
            continue
        xs, ws = (n, C, h, w_), (O, C, ks, ks)
        desc, _ = _desc(hip, xs, ws, s, d, padding)
        assert hip.conv2d_weights_plan(desc, hip.PASS_DGRAD)
        if cnt % 40 == 0:
            say(f'dgrad on Wp case {cnt}: C={C} O={O} s={s} d={d} ks={ks} pad={padding}')
        x = rs.randint(-3, 4, size=xs).astype(np.float32)
        w = rs.randint(-3, 4, size=ws).astype(np.float32)
        dy = rs.randint(-3, 4, size=(n, O, ci.OH, ci.OW)).astype(np.float32)
        ry, rdx, _ = conv2d_all(x, w, dy, s, d, padding)
        X, W, dY = DevArr(hip, x), DevArr(hip, w), DevArr(hip, dy)
        Wp = DevArr(hip, shape=(O, ks * ks, C), fill=np.nan)
        hip.conv2d_permute_weights(0, desc, W.ptr, hip.W_OIHW, Wp.ptr)
        assert np.array_equal(Wp.get(), w.reshape(O, C, ks * ks).transpose(0, 2, 1))
        beta, fill = (0, np.nan) if cnt % 2 else (1, 2.0)
        for use_wp in (False, True):
            dX = DevArr(hip, shape=xs, fill=fill)
            if use_wp:
                hip.conv2d_dgrad_pw(0, desc, dY.ptr, Wp.ptr, dX.ptr, beta)
            else:
                hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
            assert np.array_equal(dX.get() - (2.0 if beta else 0.0), rdx), (C, O, s, d, ks, padding, use_wp)
        if hip.conv2d_weights_plan(desc, hip.PASS_FWD):
            Y = DevArr(hip, shape=dy.shape, fill=np.nan)
            hip.conv2d_fwd_pw(0, desc, X.ptr, Wp.ptr, None, hip.ACT_NONE, 0.0, Y.ptr, 0)
            assert np.array_equal(Y.get(), ry), (C, O, s, d, ks, padding)
        cnt += 1
    assert cnt > 500
    # the copy itself for both source layouts: more taps than the tiled copy holds in LDS, an even tap count,
    # channel counts off and on the 64-channel blocks
    for (O, C, kh, kw) in [(3, 70, 15, 15), (5, 64, 2, 4), (2, 130, 7, 7), (33, 4, 3, 3)]:
        desc, _ = _desc(hip, (1, C, 16, 16), (O, C, kh, kw), 1, 1, 'same')
        w = rs.randint(-9, 10, size=(O, C, kh, kw)).astype(np.float32)
        want = w.reshape(O, C, kh * kw).transpose(0, 2, 1)
        for layout, src in ((hip.W_OIHW, w), (hip.W_IOHW, np.ascontiguousarray(w.transpose(1, 0, 2, 3)))):
            Wsrc, Wp = DevArr(hip, src), DevArr(hip, shape=(O, kh * kw, C), fill=np.nan)
            hip.conv2d_permute_weights(0, desc, Wsrc.ptr, layout, Wp.ptr)
            assert np.array_equal(Wp.get(), want), (O, C, kh, kw, layout)
    # geometries whose kernels do not read Wp refuse the *_pw entry points
    desc, _ = _desc(hip, (1, 3, 8, 8), (32, 3, 3, 3), 1, 1, 'same')
    assert not hip.conv2d_weights_plan(desc, hip.PASS_DGRAD) and not hip.conv2d_weights_plan(desc, hip.PASS_FWD)
    A = DevArr(hip, shape=(4096,), fill=0.0)
    with pytest.raises(hip.HipException) as e:
        hip.conv2d_dgrad_pw(0, desc, A.ptr, A.ptr, A.ptr, 0)
    assert e.value.code == hip.ERR_INVALID
    with pytest.raises(hip.HipException) as e:
        hip.conv2d_fwd_pw(0, desc, A.ptr, A.ptr, None, hip.ACT_NONE, 0.0, A.ptr, 0)
    assert e.value.code == hip.ERR_INVALID


def test_conv_remainder_units_cut_along_k_integer_exact(hip):
    """Forward and stride-1 data gradient with a few column units per workgroup and a remainder: the remainder
    units are cut into K slices, one per workgroup, and summed by a small reduction that also applies '+=' and the
    bias / activation epilogue.  Shapes with 256 q + r units (r <= 128) on the 256 compute units of the MI355X, for
    the tap-major kernels (one and two row tiles, 3x3 and 1x1) and the any-channel forward; exact on small integers."""
    rs = np.random.RandomState(63)
    cases = [((3, 64, 56, 56), (128, 64, 3, 3), 1, 1, 'same'),      # 294 units: 38 left over, 3 slices of 6 K steps
             ((5, 128, 41, 40), (256, 128, 1, 1), 1, 1, 'valid'),   # two row tiles, 1x1: 4 K steps, no cut possible
             ((2, 96, 70, 66), (160, 96, 3, 3), 1, 1, 1),           # two row tiles, ragged second; 27 K steps
             ((20, 32, 33, 31), (64, 32, 5, 5), 1, 2, 'same'),      # 64 rows: units of 64 columns
             ((4, 24, 50, 50), (96, 24, 5, 5), 1, 1, 'same'),       # any-channel forward (table gather), dgrad on Wp
             ((8, 160, 64, 72), (32, 160, 3, 3), 1, 1, (0, 1, 1, 0)),   # 32 rows: units of 128 columns
             # any-channel forward with more than 64 output channels: groups of one and three 32-column units, whose
             # last transfer per K row covers 32 columns (six and seven units per workgroup; with a K split)
             ((20, 24, 50, 50), (96, 24, 3, 3), 1, 1, 'same'), ((2, 24, 50, 50), (128, 24, 5, 5), 1, 1, 'same'),
             ((23, 20, 50, 50), (96, 20, 3, 3), 1, 1, 'valid')]
    for xs, ws, s, d, padding in cases:
        say(f'remainder units x={xs} w={ws} s={s} d={d} pad={padding}')
        desc, ci = _desc(hip, xs, ws, s, d, padding)
        O = ws[0]
        x = rs.randint(-2, 3, size=xs).astype(np.float32)
        w = rs.randint(-2, 3, size=ws).astype(np.float32)
        dy = rs.randint(-2, 3, size=(xs[0], O, ci.OH, ci.OW)).astype(np.float32)
        b = rs.randint(-3, 4, size=(O,)).astype(np.float32)
        ry, rdx, _ = conv2d_all(x, w, dy, s, d, padding)
        X, W, dY, B = DevArr(hip, x), DevArr(hip, w), DevArr(hip, dy), DevArr(hip, b)
        for beta, fill in ((0, np.nan), (1, 3.0)):
            Y = DevArr(hip, shape=dy.shape, fill=fill)
            hip.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, beta)
            assert np.array_equal(Y.get() - (3.0 if beta else 0.0), ry), (xs, ws, beta)
            dX = DevArr(hip, shape=xs, fill=fill)
            hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
            assert np.array_equal(dX.get() - (3.0 if beta else 0.0), rdx), (xs, ws, beta)
        Y = DevArr(hip, shape=dy.shape, fill=np.nan)
        hip.conv2d_fwd_bias_act(0, desc, X.ptr, W.ptr, B.ptr, hip.ACT_LEAKY_RELU, 0.25, Y.ptr)
        pre = ry + b[None, :, None, None]
        assert np.array_equal(Y.get(), np.where(pre >= 0, pre, 0.25 * pre).astype(np.float32)), (xs, ws)


def test_conv_stem_forward_from_lds_patch_integer_exact(hip):
    """Three input channels, 33-64 output channels, 3x3 (stride 1 and 2), 5x5 and 7x7 (stride 2), at least four
    tiles of 256 pixels per compute unit: the forward pass reads its B operand from an input patch in LDS (tiles of
    8 x 32 or 16 x 16 output pixels, whichever covers the plane with less overhang; blocks take tiles from a
    counter).  Planes that are whole tiles and ragged in both directions, every padding kind including asymmetric
    and none, '=' and '+=', bias and leaky ReLU in the epilogue; lnn_conv2d_fwd_path confirms that every case reaches
    the kernel.  Batches this large are slow on the CPU oracle: the first and the last image are checked against it,
    all images against the implicit-GEMM pass run on part of the batch at a time (too few tiles for the patch
    kernel), which the other tests pin to the oracle.  Exact on small integers.  Neighbouring geometries (other channel counts,
    dilation, kernel shapes, few tiles) go the implicit-GEMM way."""
    rs = np.random.RandomState(64)
    cus = hip.device_info(0)['compute_units']
    for (k, s) in [(7, 2), (5, 2), (3, 1), (3, 2)]:
        for (oh, ow, O, padding) in [(64, 64, 64, 'same'), (61, 53, 48, 'same'), (70, 40, 33, 'valid'),
                                     (93, 90, 64, (1, 0, 2, 3)), (25, 27, 40, 'same'), (130, 34, 64, 0)]:
            ih, iw = oh * s, ow * s
            if padding in ('valid', 0):
                ih, iw = ih + k - 1, iw + k - 1
            ci = info_conv2d(ih, iw, k, k, s, 1, padding)
            n = -(-4 * cus // ((ci.OH * ci.OW + 255) // 256)) + 1
            xs, ws = (n, 3, ih, iw), (O, 3, k, k)
            desc, _ = _desc(hip, xs, ws, s, 1, padding)
            assert hip.conv2d_fwd_path(desc, cus) == hip.FWD_PATH_STEM_PATCH, (xs, ws, s, padding)
            say(f'stem forward x={xs} w={ws} s={s} pad={padding} -> y {ci.OH}x{ci.OW}')
            x = rs.randint(-3, 4, size=xs).astype(np.float32)
            w = rs.randint(-3, 4, size=ws).astype(np.float32)
            b = rs.randint(-3, 4, size=(O,)).astype(np.float32)
            X, W, B = DevArr(hip, x), DevArr(hip, w), DevArr(hip, b)
            # the same convolution in batches just too small for the patch kernel
            ref = np.empty((n, O, ci.OH, ci.OW), np.float32)
            step = max(1, (4 * cus - 1) // ((ci.OH * ci.OW + 255) // 256))
            for i0 in range(0, n, step):
                m = min(step, n - i0)
                dpart, _ = _desc(hip, (m,) + xs[1:], ws, s, 1, padding)
                assert hip.conv2d_fwd_path(dpart, cus) == hip.FWD_PATH_IMPLICIT_GEMM
                Xp, Yp = DevArr(hip, x[i0:i0 + m]), DevArr(hip, shape=(m, O, ci.OH, ci.OW), fill=np.nan)
                hip.conv2d_fwd(0, dpart, Xp.ptr, W.ptr, Yp.ptr, 0)
                ref[i0:i0 + m] = Yp.get()
            for img in (0, n - 1):
                assert np.array_equal(ref[img:img + 1], conv2d_fwd(x[img:img + 1], w, s, 1, padding, dtype=np.float32))
            for beta, fill in ((0, np.nan), (1, -2.0)):
                Y = DevArr(hip, shape=ref.shape, fill=fill)
                hip.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, beta)
                assert np.array_equal(Y.get() - (-2.0 if beta else 0.0), ref), (xs, ws, s, padding, beta)
            Y = DevArr(hip, shape=ref.shape, fill=np.nan)
            hip.conv2d_fwd_bias_act(0, desc, X.ptr, W.ptr, B.ptr, hip.ACT_LEAKY_RELU, 0.25, Y.ptr)
            pre = ref + b[None, :, None, None]
            assert np.array_equal(Y.get(), np.where(pre >= 0, pre, 0.25 * pre).astype(np.float32)), (xs, ws, s, padding)
            # weight gradient (the patch kernel where OW % 4 == 0): the whole batch in one call against the same
            # batches accumulated with '+=' on the implicit-GEMM pass, whose first image is pinned to the oracle
            dy = rs.randint(-3, 4, size=ref.shape).astype(np.float32)
            dY = DevArr(hip, dy)
            dWref = DevArr(hip, shape=ws, fill=0.0)
            for i0 in range(0, n, step):
                m = min(step, n - i0)
                dpart, _ = _desc(hip, (m,) + xs[1:], ws, s, 1, padding)
                Xp, dYp = DevArr(hip, x[i0:i0 + m]), DevArr(hip, dy[i0:i0 + m])
                hip.conv2d_wgrad(0, dpart, Xp.ptr, dYp.ptr, dWref.ptr, 1)
            done, _ = _desc(hip, (1,) + xs[1:], ws, s, 1, padding)
            dW1 = DevArr(hip, shape=ws, fill=np.nan)
            X1, dY1 = DevArr(hip, x[:1]), DevArr(hip, dy[:1])
            hip.conv2d_wgrad(0, done, X1.ptr, dY1.ptr, dW1.ptr, 0)
            assert np.array_equal(dW1.get(), conv2d_dw(x[:1], dy[:1], ws, s, 1, padding))
            for beta, fill in ((0, np.nan), (1, 5.0)):
                dW = DevArr(hip, shape=ws, fill=fill)
                hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, beta)
                assert np.array_equal(dW.get() - (5.0 if beta else 0.0), dWref.get()), (xs, ws, s, padding, beta)
    # neighbours of the stem geometries stay on the other kernels
    for xs, ws, s, d in [((70, 3, 128, 128), (32, 3, 7, 7), 2, 1), ((70, 3, 64, 64), (96, 3, 3, 3), 1, 1),
                         ((70, 4, 128, 128), (64, 4, 5, 5), 2, 1), ((70, 3, 64, 64), (64, 3, 3, 3), 1, 2),
                         ((70, 3, 64, 64), (64, 3, 3, 5), 1, 1), ((70, 3, 64, 64), (64, 3, 5, 5), 1, 1),
                         ((8, 3, 128, 128), (64, 3, 7, 7), 2, 1)]:
        desc, _ = _desc(hip, xs, ws, s, d, 'same')
        assert hip.conv2d_fwd_path(desc, 256) == hip.FWD_PATH_IMPLICIT_GEMM, (xs, ws, s, d)
    # float data at a stem's real size against the fp64 restatement (first and last image)
    xs, ws = (24, 3, 224, 224), (64, 3, 7, 7)
    desc, ci = _desc(hip, xs, ws, 2, 1, 'same')
    assert cus != 256 or hip.conv2d_fwd_path(desc, cus) == hip.FWD_PATH_STEM_PATCH
    x = rs.uniform(-1, 1, size=xs).astype(np.float32)
    w = rs.uniform(-1, 1, size=ws).astype(np.float32)
    X, W = DevArr(hip, x), DevArr(hip, w)
    Y = DevArr(hip, shape=(xs[0], 64, ci.OH, ci.OW), fill=np.nan)
    hip.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, 0)
    y = Y.get()
    for img in (0, xs[0] - 1):
        assert rel_err(y[img:img + 1], conv2d_fwd(x[img:img + 1], w, 2, 1, 'same')) <= TOL


def test_conv_stem_dgrad_parity_rows_integer_exact(hip):
    """Stride 2, at most 4 input channels, 32 or more output channels (a multiple of 8), at least two tiles of 32 x 32
    input pixels per compute unit: the data gradient computes the four pixel parities of each channel as rows of a
    16-row GEMM over a dY patch in LDS (v_mfma_f32_16x16x4_f32).  Kernels from 2 x 2 to 8 x 8 (square and not), every
    padding kind, image sizes that are not multiples of the tile and odd, '=' and '+='; lnn_conv2d_dgrad_path confirms
    the path.  The first and the last image are checked against the oracle, all images against the same call on
    batches too small for this kernel (the vector-ALU or the implicit-GEMM data gradient, pinned by the other tests).
    Exact on small integers."""
    rs = np.random.RandomState(65)
    cus = hip.device_info(0)['compute_units']
    cases = [(3, 64, 7, 7, 3, 70, 66), (3, 32, 5, 5, 'same', 70, 66), (4, 40, 3, 3, 'same', 64, 64), (1, 64, 7, 7, 'valid', 71, 67),
             (3, 48, 4, 4, 1, 65, 33), (2, 32, 8, 8, (2, 2, 4, 3), 70, 66), (3, 64, 2, 2, 0, 70, 66), (3, 32, 6, 3, (1, 0, 0, 2), 33, 130),
             (4, 64, 7, 5, (2, 3, 1, 0), 70, 66), (3, 72, 5, 5, 2, 37, 41)]
    for C, O, kh, kw, padding, ih, iw in cases:
        tiles_per_img = (((ih + 1) // 2 + 15) // 16) * (((iw + 1) // 2 + 15) // 16)
        n = -(-2 * cus // tiles_per_img) + 1
        xs, ws = (n, C, ih, iw), (O, C, kh, kw)
        ci = info_conv2d(ih, iw, kh, kw, 2, 1, padding)
        desc = hip.conv_desc(n, C, ih, iw, O, kh, kw, ci.OH, ci.OW, ci.PADL, ci.PADT, 2, 1)
        assert hip.conv2d_dgrad_path(desc, 0, cus)[0] == hip.DGRAD_PATH_STEM_MFMA, (xs, ws, padding)
        say(f'stem dgrad x={xs} w={ws} pad={padding} dy {ci.OH}x{ci.OW}')
        w = rs.randint(-3, 4, size=ws).astype(np.float32)
        dy = rs.randint(-3, 4, size=(n, O, ci.OH, ci.OW)).astype(np.float32)
        W, dY = DevArr(hip, w), DevArr(hip, dy)
        ref = np.empty(xs, np.float32)
        step = max(1, (2 * cus - 1) // tiles_per_img)
        for i0 in range(0, n, step):
            m = min(step, n - i0)
            dpart = hip.conv_desc(m, C, ih, iw, O, kh, kw, ci.OH, ci.OW, ci.PADL, ci.PADT, 2, 1)
            assert hip.conv2d_dgrad_path(dpart, 0, cus)[0] != hip.DGRAD_PATH_STEM_MFMA
            dYp, dXp = DevArr(hip, dy[i0:i0 + m]), DevArr(hip, shape=(m,) + xs[1:], fill=np.nan)
            hip.conv2d_dgrad(0, dpart, dYp.ptr, W.ptr, dXp.ptr, 0)
            ref[i0:i0 + m] = dXp.get()
        for img in (0, n - 1):
            assert np.array_equal(ref[img:img + 1], conv2d_dx(dy[img:img + 1], w, (1,) + xs[1:], 2, 1, padding)), (xs, ws, padding)
        for beta, fill in ((0, np.nan), (1, 3.0)):
            dX = DevArr(hip, shape=xs, fill=fill)
            hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
            assert np.array_equal(dX.get() - (3.0 if beta else 0.0), ref), (xs, ws, padding, beta)
    # neighbours that stay on the other kernels: few output channels, not a multiple of 8, stride 1, dilation, five
    # channels, a 9 x 9 kernel and an 8 x 8 one with odd padding (five dY rows per pixel pair), too few tiles
    for (N, C, O, k, s, d) in [(64, 3, 16, 7, 2, 1), (64, 3, 36, 7, 2, 1), (64, 3, 64, 3, 1, 1), (64, 3, 64, 3, 2, 2),
                               (64, 5, 64, 7, 2, 1), (64, 3, 64, 9, 2, 1), (64, 3, 64, 8, 2, 1), (8, 3, 64, 7, 2, 1)]:
        ci = info_conv2d(70, 66, k, k, s, d, 'same')
        desc = hip.conv_desc(N, C, 70, 66, O, k, k, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)
        assert hip.conv2d_dgrad_path(desc, 0, 256)[0] != hip.DGRAD_PATH_STEM_MFMA, (N, C, O, k, s, d)


def test_conv_passes_on_weights_with_swapped_channel_axes(hip):
    """A transposed convolution keeps its kernel as [C][O][KH][KW] relative to the convolution whose passes it
    borrows.  lnn_conv2d_permute_weights_f32(LNN_W_IOHW) makes Wp straight from that storage, the *_pw passes run
    on it, and lnn_conv2d_wgrad_iohw_f32 writes the weight gradient in that storage ('=' and '+=', split-K
    reduction and direct epilogue), all exact against the oracle on the explicitly swapped kernel."""
    rs = np.random.RandomState(62)
    cases = [((2, 64, 12, 12), (64, 64, 5, 5), 2, 1, 2), ((3, 128, 9, 10), (32, 128, 3, 3), 1, 1, 'same'),
             ((2, 128, 8, 8), (160, 128, 3, 3), 1, 2, 'same'), ((1, 32, 20, 20), (96, 32, 1, 1), 1, 1, 'valid'),
             ((16, 128, 32, 32), (256, 128, 5, 5), 2, 1, 2), ((2, 64, 6, 33), (40, 64, 2, 2), 1, 1, 'valid'),
             # few or odd channel counts: the weight-gradient kernel whose column groups span taps
             ((4, 32, 20, 20), (8, 32, 3, 3), 1, 1, 'same'), ((2, 96, 14, 16), (40, 96, 3, 3), 2, 1, 1),
             ((3, 32, 9, 14), (130, 32, 5, 5), 1, 1, 2)]
    for xs, ws, s, d, padding in cases:
        say(f'swapped-axes weights x={xs} w={ws} s={s} d={d} pad={padding}')
        desc, ci = _desc(hip, xs, ws, s, d, padding)
        O, C, KH, KW = ws
        x = rs.randint(-2, 3, size=xs).astype(np.float32)
        w = rs.randint(-2, 3, size=ws).astype(np.float32)
        dy = rs.randint(-2, 3, size=(xs[0], O, ci.OH, ci.OW)).astype(np.float32)
        ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
        w_io = np.ascontiguousarray(w.transpose(1, 0, 2, 3))          # how the caller stores it
        X, Wio, dY = DevArr(hip, x), DevArr(hip, w_io), DevArr(hip, dy)
        Wp = DevArr(hip, shape=(O, KH * KW, C), fill=np.nan)
        hip.conv2d_permute_weights(0, desc, Wio.ptr, hip.W_IOHW, Wp.ptr)
        assert np.array_equal(Wp.get(), w.reshape(O, C, KH * KW).transpose(0, 2, 1))
        assert hip.conv2d_weights_plan(desc, hip.PASS_FWD) and hip.conv2d_weights_plan(desc, hip.PASS_WGRAD)
        Y = DevArr(hip, shape=dy.shape, fill=np.nan)
        hip.conv2d_fwd_pw(0, desc, X.ptr, Wp.ptr, None, hip.ACT_NONE, 0.0, Y.ptr, 0)
        assert np.array_equal(Y.get(), ry)
        if hip.conv2d_weights_plan(desc, hip.PASS_DGRAD):
            dX = DevArr(hip, shape=xs, fill=1.0)
            hip.conv2d_dgrad_pw(0, desc, dY.ptr, Wp.ptr, dX.ptr, 1)
            assert np.array_equal(dX.get() - 1.0, rdx)
        for beta, fill in ((0, np.nan), (1, -3.0)):
            dWio = DevArr(hip, shape=w_io.shape, fill=fill)
            hip.conv2d_wgrad_iohw(0, desc, X.ptr, dY.ptr, dWio.ptr, beta)
            assert np.array_equal(dWio.get() - (-3.0 if beta else 0.0), rdw.transpose(1, 0, 2, 3)), (xs, ws, beta)
    # output planes smaller than a K step stay on the table-driven weight-gradient kernel, which cannot write swapped axes
    desc, _ = _desc(hip, (1, 3, 4, 4), (8, 3, 3, 3), 1, 1, 'same')
    assert not hip.conv2d_weights_plan(desc, hip.PASS_WGRAD)
    A = DevArr(hip, shape=(4096,), fill=0.0)
    with pytest.raises(hip.HipException) as e:
        hip.conv2d_wgrad_iohw(0, desc, A.ptr, A.ptr, A.ptr, 0)
    assert e.value.code == hip.ERR_UNSUPPORTED


def test_conv_few_tiles_split_k_integer_exact(hip):
    """Deep layers on small images have a long K and few output tiles: forward
    and dgrad then split K over the idle compute units and a second kernel
    sums the slices into the NCHW (or class-strided) output.  Exact on
    integers, with and without accumulation, stride 1 and 2, channel counts on
    and off the multiple-of-32 kernels."""
    rs = np.random.RandomState(31)
    cases = [((2, 128, 16, 16), (256, 128, 5, 5), 2, 1, 2), ((2, 256, 8, 8), (512, 256, 5, 5), 2, 1, 2),
             ((1, 256, 6, 6), (96, 256, 3, 3), 1, 1, 'same'), ((3, 130, 5, 7), (70, 130, 3, 3), 1, 1, 'same'),
             ((1, 512, 4, 4), (40, 512, 1, 1), 1, 1, 'valid'), ((2, 96, 9, 9), (33, 96, 3, 3), 3, 2, 'same')]
    for i, (xs, ws, s, d, padding) in enumerate(cases):
        say(f'conv split-K x={xs} w={ws} s={s} d={d} pad={padding}')
        x = rs.randint(4, size=xs).astype(np.float32)
        w = rs.randint(4, size=ws).astype(np.float32)
        ci = info_conv2d(xs[2], xs[3], ws[2], ws[3], s, d, padding)
        dy = rs.randint(4, size=(xs[0], ws[0], ci.OH, ci.OW)).astype(np.float32)
        ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
        for prefill in (None, 5.0):
            y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding, prefill=prefill)
            off = 0.0 if prefill is None else prefill
            assert np.array_equal(y, ry), ('fwd', xs, ws)
            assert np.array_equal(dx - off, rdx), ('dX', xs, ws)
            assert np.array_equal(dw - off, rdw), ('dW', xs, ws)


def test_conv_wgrad_equal_k_shares_integer_exact(hip):
    """Weight gradients whose whole sub-tiles times K slices would leave a fifth of the chip idle (256 -> 512 channels
    5x5 at 8 x 8 output pixels: 200 sub-tiles of 16 K steps on 256 compute units) deal the K steps of all sub-tiles
    out in equal runs that cross sub-tile borders; a run's two pieces go to blocks of their own and the slice sum
    adds each sub-tile's two or three blocks.  lnn_conv2d_wgrad_last_plan confirms the plan; exact on integers, '='
    into NaN and '+=', OIHW and channel-swapped storage, and the allocation-free entry point (whose fixed array the
    blocks fill exactly) bit for bit the same."""
    rs = np.random.RandomState(41)
    cus = hip.device_info(0)['compute_units']
    cases = [((16, 256, 16, 16), (512, 256, 5, 5), 2, 1, 2), ((16, 512, 8, 8), (512, 512, 3, 3), 1, 1, 'same'),
             ((16, 256, 8, 8), (500, 256, 5, 5), 1, 1, 'same')]
    for xs, ws, s, d, padding in cases:
        say(f'wgrad equal K shares x={xs} w={ws} s={s} pad={padding}')
        desc, ci = _desc(hip, xs, ws, s, d, padding)
        x = rs.randint(4, size=xs).astype(np.float32)
        dy = (rs.randint(4, size=(xs[0], ws[0], ci.OH, ci.OW)) - 1).astype(np.float32)
        rdw = np.zeros(ws, np.float64)
        for i0 in range(0, xs[0], 4):
            rdw += conv2d_dw(x[i0:i0 + 4], dy[i0:i0 + 4], ws, s, d, padding)
        X, dY = DevArr(hip, x), DevArr(hip, dy)
        dW = DevArr(hip, shape=ws, fill=np.nan)
        hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, 0)
        plan = hip.conv2d_wgrad_last_plan(0)
        if cus == 256:
            assert plan[2] == 1 and plan[0] == cus, (plan, xs, ws)
        got = dW.get()
        assert np.array_equal(got, rdw), ('dW =', xs, ws)
        w0 = rs.randint(-3, 4, size=ws).astype(np.float32)
        dW2 = DevArr(hip, w0)
        hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW2.ptr, 1)
        assert np.array_equal(dW2.get(), rdw + w0), ('dW +=', xs, ws)
        dW3 = DevArr(hip, shape=(ws[1], ws[0], ws[2], ws[3]), fill=np.nan)
        hip.conv2d_wgrad_iohw(0, desc, X.ptr, dY.ptr, dW3.ptr, 0)
        assert np.array_equal(dW3.get(), rdw.transpose(1, 0, 2, 3)), ('dW swapped', xs, ws)
        dW4 = DevArr(hip, shape=ws, fill=np.nan)
        hip.conv2d_wgrad_noalloc(0, desc, X.ptr, dY.ptr, dW4.ptr, 0)
        assert hip.conv2d_wgrad_last_plan(0) == plan
        assert np.array_equal(dW4.get(), got), ('dW without allocation', xs, ws)


def test_conv_fwd_bias_act_matches_separate_kernels(hip):
    """Fused forward through the C ABI against the three separate launches
    (convolution, broadcast bias add, leaky ReLU) of the same library, bit for
    bit on random float data, on the direct, table-driven and split-K paths;
    bias only, activation only, both."""
    rs = np.random.RandomState(41)
    cases = [((2, 128, 12, 12), (128, 128, 3, 3), 1, 1, 'same'), ((2, 3, 17, 9), (5, 3, 3, 3), 2, 1, 1),
             ((1, 256, 6, 6), (96, 256, 3, 3), 1, 1, 'same'), ((2, 64, 9, 11), (40, 64, 1, 1), 1, 1, 'valid')]
    for xs, ws, s, d, padding in cases:
        say(f'conv fused x={xs} w={ws} s={s} pad={padding}')
        desc, ci = _desc(hip, xs, ws, s, d, padding)
        x = rs.normal(0, 1, xs).astype(np.float32)
        w = rs.normal(0, 1, ws).astype(np.float32)
        b = rs.normal(0, 3, (ws[0],)).astype(np.float32)
        ys = (xs[0], ws[0], ci.OH, ci.OW)
        X, W, B = DevArr(hip, x), DevArr(hip, w), DevArr(hip, b)
        Y0, Y1, Y2 = (DevArr(hip, shape=ys, fill=np.nan) for _ in range(3))
        hip.conv2d_fwd(0, desc, X.ptr, W.ptr, Y0.ptr, 0)
        n = int(np.prod(ys))
        for use_b, act in ((True, hip.ACT_LEAKY_RELU), (True, hip.ACT_NONE), (False, hip.ACT_LEAKY_RELU)):
            ref = Y0.get()
            if use_b:
                ref = ref + b.reshape(1, -1, 1, 1)
            if act == hip.ACT_LEAKY_RELU:
                ref = np.where(ref >= 0, ref, np.float32(0.1) * ref)
            hip.conv2d_fwd_bias_act(0, desc, X.ptr, W.ptr, B.ptr if use_b else None, act, 0.1, Y1.ptr)
            assert np.array_equal(Y1.get(), ref.astype(np.float32)), (xs, ws, use_b, act)
        # and against the library's own separate kernels
        hip.binary_bcast(0, hip.BIN_ADD, ys, ys, (1, ws[0], 1, 1), Y0.ptr, B.ptr, Y2.ptr, 0)
        hip.ew_fwd(0, hip.EW_LEAKY_RELU, n, Y2.ptr, Y2.ptr, 0.1, 0)
        hip.conv2d_fwd_bias_act(0, desc, X.ptr, W.ptr, B.ptr, hip.ACT_LEAKY_RELU, 0.1, Y1.ptr)
        assert np.array_equal(Y1.get(), Y2.get()), (xs, ws)
    with pytest.raises(hip.HipException):
        hip.conv2d_fwd_bias_act(0, desc, X.ptr, W.ptr, B.ptr, 7, 0.1, Y1.ptr)


def test_depthwise_integer_exact_and_float(hip):
    """Depthwise forward / dgrad / wgrad through the C ABI: integer-exact over
    strides, dilations, kernel sizes and paddings with '=' and '+=', then a
    larger float case within tolerance (the kernel gradient sums tens of
    thousands of products per tap)."""
    rs = np.random.RandomState(51)
    cnt = 0
    grid = list(itertools.product((1, 2, 3), (1, 2), (1, 2, 3, 5), ('same', 'valid', 1, (2, 0, 1, 3)),
                                  ((2, 3, 11, 9), (1, 70, 6, 7))))
    # rows too wide for the small LDS band (the one-block-per-CU variant), and a 7x7 filter
    grid += [(1, 1, 3, 'same', (1, 2, 12, 1500)), (2, 1, 5, 'same', (1, 2, 9, 2100)), (1, 2, 7, 'same', (2, 3, 20, 20)),
             (2, 1, 7, 3, (1, 2, 30, 700))]
    for s, d, ks, padding, xs in grid:
        try:
            ci = info_conv2d(xs[2], xs[3], ks, ks, s, d, padding)
        except ValueError:
            continue
        if ci.OH <= 0 or ci.OW <= 0:
            continue
        if cnt % 40 == 0:
            say(f'depthwise case {cnt}: x={xs} ks={ks} s={s} d={d} pad={padding}')
        x = rs.randint(-4, 5, size=xs).astype(np.float32)
        k = rs.randint(-4, 5, size=(xs[1], ks, ks)).astype(np.float32)
        dy = rs.randint(-4, 5, size=(xs[0], xs[1], ci.OH, ci.OW)).astype(np.float32)
        ry, rdx, rdk = depthwise_all(x, k, dy, s, d, padding)
        desc = hip.conv_desc(xs[0], xs[1], xs[2], xs[3], xs[1], ks, ks, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)
        pre = None if cnt % 2 else 2.0
        X, K, dY = DevArr(hip, x), DevArr(hip, k), DevArr(hip, dy)
        Y = DevArr(hip, shape=dy.shape, fill=np.nan)
        dX = DevArr(hip, shape=xs, fill=np.nan if pre is None else pre)
        dK = DevArr(hip, shape=k.shape, fill=np.nan if pre is None else pre)
        beta = 0 if pre is None else 1
        hip.depthwise_conv2d_fwd(0, desc, X.ptr, K.ptr, Y.ptr, 0)
        hip.depthwise_conv2d_dgrad(0, desc, dY.ptr, K.ptr, dX.ptr, beta)
        hip.depthwise_conv2d_wgrad(0, desc, X.ptr, dY.ptr, dK.ptr, beta)
        off = 0.0 if pre is None else pre
        assert np.array_equal(Y.get(), ry), ('fwd', xs, ks, s, d, padding)
        assert np.array_equal(dX.get() - off, rdx), ('dX', xs, ks, s, d, padding)
        assert np.array_equal(dK.get() - off, rdk), ('dK', xs, ks, s, d, padding)
        cnt += 1
    assert cnt > 150
    xs, ks = (4, 96, 56, 56), 3
    say(f'depthwise float x={xs}')
    ci = info_conv2d(56, 56, ks, ks, 1, 1, 'same')
    x = rs.normal(0, 1, xs).astype(np.float32)
    k = rs.normal(0, 1, (96, ks, ks)).astype(np.float32)
    dy = rs.normal(0, 1, xs).astype(np.float32)
    ry, rdx, rdk = depthwise_all(x, k, dy, 1, 1, 'same')
    desc = hip.conv_desc(4, 96, 56, 56, 96, ks, ks, 56, 56, ci.PADL, ci.PADT, 1, 1)
    X, K, dY = DevArr(hip, x), DevArr(hip, k), DevArr(hip, dy)
    Y, dX, dK = DevArr(hip, shape=xs, fill=np.nan), DevArr(hip, shape=xs, fill=np.nan), DevArr(hip, shape=k.shape, fill=np.nan)
    hip.depthwise_conv2d_fwd(0, desc, X.ptr, K.ptr, Y.ptr, 0)
    hip.depthwise_conv2d_dgrad(0, desc, dY.ptr, K.ptr, dX.ptr, 0)
    hip.depthwise_conv2d_wgrad(0, desc, X.ptr, dY.ptr, dK.ptr, 0)
    assert rel_err(Y.get(), ry) <= TOL and rel_err(dX.get(), rdx) <= TOL and rel_err(dK.get(), rdk) <= TOL
    bad = hip.conv_desc(4, 96, 56, 56, 64, ks, ks, 56, 56, 1, 1, 1, 1)
    with pytest.raises(hip.HipException):
        hip.depthwise_conv2d_fwd(0, bad, X.ptr, K.ptr, Y.ptr, 0)


# benchmark geometries at a reduced batch (the oracle materialises im2col in fp64)
_BENCH = {
    'cfg1': ((8, 3, 64, 64), (32, 3, 3, 3), 1, 1, 'same', 0),
    'cfg3': ((2, 128, 56, 56), (128, 128, 3, 3), 1, 1, 'same', 0),
    'cfg4a': ((2, 3, 224, 224), (64, 3, 7, 7), 2, 1, 3, 0),
    'cfg4b': ((4, 256, 28, 28), (512, 256, 1, 1), 1, 1, 'same', 1),
    'cfg4c': ((2, 64, 64, 64), (64, 64, 3, 3), 1, 2, 2, 2),
    'cfg5_L1': ((2, 3, 128, 128), (64, 3, 5, 5), 2, 1, 2, 0),
    'cfg5_L2': ((2, 64, 64, 64), (128, 64, 5, 5), 2, 1, 2, 0),
    'cfg5_L3': ((4, 128, 32, 32), (256, 128, 5, 5), 2, 1, 2, 0),
    'cfg5_L4': ((8, 256, 16, 16), (512, 256, 5, 5), 2, 1, 2, 0),
}


@pytest.mark.parametrize('name', list(_BENCH))
def test_conv_benchmark_geometries_float(hip, name):
    xs, ws, s, d, padding, seed = _BENCH[name]
    rs = np.random.RandomState(seed)
    x = rs.uniform(-1, 1, xs).astype(np.float32)
    w = rs.normal(0, np.sqrt(2.0 / (ws[1] * ws[2] * ws[3])), ws).astype(np.float32)
    ci = info_conv2d(xs[2], xs[3], ws[2], ws[3], s, d, padding)
    dy = rs.normal(0, 1, (xs[0], ws[0], ci.OH, ci.OW)).astype(np.float32)
    say(f'conv {name} x={xs} w={ws} s={s} d={d} pad={padding}')
    y, dx, dw = _run_conv(hip, x, w, dy, s, d, padding)
    ry, rdx, rdw = conv2d_all(x, w, dy, s, d, padding)
    errs = (rel_err(y, ry), rel_err(dx, rdx), rel_err(dw, rdw))
    say(f'  normalised errors fwd/dX/dW = {errs}')
    assert max(errs) <= TOL


def test_multi_tensor_updates_equal_single_launches(hip):
    """lnn_sgd_update_multi_f32 / lnn_adam_update_multi_f32 against one call per tensor: the same bits, for more
    tensors than one launch holds and with an empty tensor among them."""
    rs = np.random.RandomState(77)
    sizes = [1, 7, 0, 300, 4097, 64 * 9, 33, 1 << 16] + [11 + 3 * i for i in range(14)]   # 22 tensors
    mk = lambda: [rs.standard_normal(max(n, 1)).astype(np.float32) for n in sizes]
    v0, g0, a0, b0 = mk(), mk(), mk(), [np.abs(x) for x in mk()]
    for kind in ('sgd', 'sgd_nesterov', 'adam'):
        say(f'multi-tensor update {kind}')
        one = [[DevArr(hip, x) for x in arrs] for arrs in (v0, g0, a0, b0)]
        many = [[DevArr(hip, x) for x in arrs] for arrs in (v0, g0, a0, b0)]
        for i, n in enumerate(sizes):
            if kind == 'adam':
                hip.adam_update(0, n, one[0][i].ptr, one[1][i].ptr, one[2][i].ptr, one[3][i].ptr, 0.9, 0.999, 1e-2)
            else:
                hip.sgd_update(0, n, one[0][i].ptr, one[1][i].ptr, one[2][i].ptr, 0.9, 1e-2, kind == 'sgd_nesterov')
        ptrs = [[d.ptr for d in col] for col in many]
        if kind == 'adam':
            hip.adam_update_multi(0, sizes, ptrs[0], ptrs[1], ptrs[2], ptrs[3], 0.9, 0.999, 1e-2)
        else:
            hip.sgd_update_multi(0, sizes, ptrs[0], ptrs[1], ptrs[2], 0.9, 1e-2, kind == 'sgd_nesterov')
        for col_one, col_many in zip(one, many):
            for x, y in zip(col_one, col_many):
                assert np.array_equal(x.get(), y.get())
    hip.sgd_update_multi(0, [], [], [], [], 0.9, 1e-2, False)      # nothing to do
    with pytest.raises(hip.HipException):
        hip.sgd_update_multi(0, [4], [None], [many[1][0].ptr], [many[2][0].ptr], 0.9, 1e-2, False)


def test_multi_tensor_updates_refresh_permuted_copies(hip):
    """lnn_sgd_update_multi_wp_f32 / lnn_adam_update_multi_wp_f32: the same new values and optimizer state as the
    plain multi-tensor calls, bit for bit, and for every tensor that brings a permuted copy the copy equals
    Wp[o][tap][c] of the new values, for tensors stored [O][C][taps] and [C][O][taps]; tensors without a copy, an empty tensor and more tensors than one launch holds
    among them.  A copy whose channel and tap counts do not divide the tensor is refused."""
    rs = np.random.RandomState(78)
    # (O, C, KK); [O][C][taps] tensors with fewer than 64 channels, a ragged last run of 64, whole runs, and taps x 64
    # beyond what the kernel stages at once
    shapes = ([(32, 32, 9), None, (64, 3, 49), (5, 7, 1), None, (40, 24, 25), (8, 130, 4), (6, 130, 9), (4, 64, 25),
               (2, 200, 16), (2, 64, 81)] + [None] * 8 + [(3, 5, 6)])
    lays = ([hip.W_OIHW, 0, hip.W_IOHW, hip.W_IOHW, 0, hip.W_OIHW, hip.W_IOHW] + [hip.W_OIHW] * 4 + [0] * 8
            + [hip.W_IOHW])
    sizes = [int(np.prod(sh)) if sh else 37 + i for i, sh in enumerate(shapes)]
    sizes[4] = 0
    mk = lambda: [rs.standard_normal(max(n, 1)).astype(np.float32) for n in sizes]
    v0, g0, a0, b0 = mk(), mk(), mk(), [np.abs(x) for x in mk()]
    cs = [sh[1] if sh else 0 for sh in shapes]
    kks = [sh[2] if sh else 0 for sh in shapes]
    for kind in ('sgd', 'sgd_nesterov', 'sgd_no_momentum', 'adam'):
        say(f'multi-tensor update with permuted copies {kind}')
        mom = 0.0 if kind == 'sgd_no_momentum' else 0.9
        plain = [[DevArr(hip, x) for x in arrs] for arrs in (v0, g0, a0, b0)]
        fused = [[DevArr(hip, x) for x in arrs] for arrs in (v0, g0, a0, b0)]
        wps = [DevArr(hip, shape=(n,), fill=np.nan) if sh else None for sh, n in zip(shapes, sizes)]
        pp, pf = [[d.ptr for d in col] for col in plain], [[d.ptr for d in col] for col in fused]
        wptrs = [w.ptr if w is not None else None for w in wps]
        if kind == 'adam':
            hip.adam_update_multi(0, sizes, pp[0], pp[1], pp[2], pp[3], 0.9, 0.999, 1e-2)
            hip.adam_update_multi_wp(0, sizes, pf[0], pf[1], pf[2], pf[3], 0.9, 0.999, 1e-2, wptrs, cs, kks, lays)
        else:
            hip.sgd_update_multi(0, sizes, pp[0], pp[1], pp[2], mom, 1e-2, kind == 'sgd_nesterov')
            hip.sgd_update_multi_wp(0, sizes, pf[0], pf[1], pf[2], mom, 1e-2, kind == 'sgd_nesterov', wptrs, cs, kks, lays)
            if mom == 0.0:   # the accumulator's old value is not read: the new one is -lr * g
                for acc, g, n in zip(fused[2], g0, sizes):
                    assert n == 0 or np.array_equal(acc.get(), np.float32(-1e-2) * g)
        for col_p, col_f in zip(plain, fused):
            for x, y in zip(col_p, col_f):
                assert np.array_equal(x.get(), y.get())
        for sh, lay, w, v in zip(shapes, lays, wps, fused[0]):
            if sh:   # the tensor is stored [O][C][KK], or [C][O][KK] with swapped channel axes
                O, C, KK = sh
                want = v.get().reshape(O, C, KK).transpose(0, 2, 1) if lay == hip.W_OIHW else v.get().reshape(C, O, KK).transpose(1, 2, 0)
                assert np.array_equal(w.get().reshape(O, KK, C), want), (kind, sh, lay)
    with pytest.raises(hip.HipException) as e:
        hip.sgd_update_multi_wp(0, [10], [fused[0][0].ptr], [fused[1][0].ptr], [fused[2][0].ptr], 0.9, 1e-2, False,
                                [wps[0].ptr], [3], [3])
    assert e.value.code == hip.ERR_INVALID


def test_bias_act_bwd_one_pass(hip):
    """dpre = dy * f'(y) and dbias[o] (+)= sum dpre: exact on small integers with a power-of-two slope, <= 1e-5 of
    the largest |dbias| on floats (fp32 sums against fp64)."""
    rs = np.random.RandomState(21)
    cases = [(1, 1, 1), (2, 3, 7), (4, 8, 56 * 56), (3, 5, 2048), (2, 4, 2049 * 4), (1, 2, 5000), (5, 130, 36),
             (64, 16, 32 * 32), (1, 300, 3), (4, 300, 64), (2, 512, 100), (16, 256, 256)]
    for N, O, HW in cases:
        for act, slope in [(hip.ACT_LEAKY_RELU, 0.25), (hip.ACT_NONE, 0.0)]:
            say(f'bias_act_bwd N={N} O={O} HW={HW} act={act}')
            y = rs.randint(-8, 8, size=(N, O, HW)).astype(np.float32)
            dy = rs.randint(-8, 8, size=(N, O, HW)).astype(np.float32)
            b0 = rs.randint(-8, 8, size=(O,)).astype(np.float32)
            ref = dy * (np.where(y >= 0, 1.0, slope).astype(np.float32) if act == hip.ACT_LEAKY_RELU else 1.0)
            rb = ref.astype(np.float64).sum(axis=(0, 2))
            Y, DY = DevArr(hip, y), DevArr(hip, dy)
            P, B = DevArr(hip, shape=y.shape, fill=np.nan), DevArr(hip, b0)
            hip.bias_act_bwd(0, N, O, HW, Y.ptr, DY.ptr, act, slope, P.ptr, B.ptr, 1)
            assert np.array_equal(P.get(), ref)
            assert np.array_equal(B.get(), (rb + b0).astype(np.float32))
            hip.bias_act_bwd(0, N, O, HW, Y.ptr, DY.ptr, act, slope, None, B.ptr, 0)       # bias gradient only
            assert np.array_equal(B.get(), rb.astype(np.float32))
            hip.bias_act_bwd(0, N, O, HW, Y.ptr, DY.ptr, act, slope, DY.ptr, None, 0)      # in place, no bias
            assert np.array_equal(DY.get(), ref)
    N, O, HW = 32, 128, 56 * 56
    y = rs.standard_normal((N, O, HW)).astype(np.float32)
    dy = rs.standard_normal((N, O, HW)).astype(np.float32)
    ref = dy.astype(np.float64) * np.where(y >= 0, 1.0, np.float64(np.float32(0.2)))
    Y, DY = DevArr(hip, y), DevArr(hip, dy)
    P, B = DevArr(hip, shape=y.shape, fill=np.nan), DevArr(hip, shape=(O,), fill=np.nan)
    hip.bias_act_bwd(0, N, O, HW, Y.ptr, DY.ptr, hip.ACT_LEAKY_RELU, 0.2, P.ptr, B.ptr, 0)
    assert rel_err(P.get(), ref) <= 1e-6
    assert rel_err(B.get(), ref.sum(axis=(0, 2))) <= 1e-5
    for bad in [lambda: hip.bias_act_bwd(0, 0, 1, 1, Y.ptr, DY.ptr, hip.ACT_NONE, 0.0, P.ptr, B.ptr, 0),
                lambda: hip.bias_act_bwd(0, 1, 1, 1, Y.ptr, DY.ptr, 7, 0.0, P.ptr, B.ptr, 0),
                lambda: hip.bias_act_bwd(0, 1, 1, 1, Y.ptr, DY.ptr, hip.ACT_NONE, 0.0, None, None, 0),
                lambda: hip.bias_act_bwd(0, 1, 1, 1, None, DY.ptr, hip.ACT_LEAKY_RELU, 0.1, P.ptr, None, 0)]:
        with pytest.raises(hip.HipException):
            bad()


def test_random_initialisers_match_the_counter_hash(hip):
    """Integer stream bit for bit: with low 0 and span 1 the output IS (float)hash * 2^-32.  The affine map is one
    single-precision fused multiply-add on both sides (the reference's kernels are built with
    -cl-single-precision-constant, CLDevice.py:93), so the uniform initialiser is bit-exact for any bounds;
    Box-Muller goes through single-precision log / cos, whose last bits differ between libraries: 2e-6 of
    stddev-scaled absolute error."""
    for n, seed in [(1, 0), (255, 1), (100003, 2147483647), (1 << 20, 123456789), (70000, 0xFFFFFFF0)]:
        say(f'random n={n} seed={seed}')
        out = DevArr(hip, shape=(n,), fill=np.nan)
        hip.random_uniform(0, out.ptr, n, seed, 0.0, 1.0)
        assert np.array_equal(out.get(), hash_rng.random_uniform(n, seed, 0.0, 1.0))
        hip.random_uniform(0, out.ptr, n, seed, -0.3, 0.9)
        ref = hash_rng.random_uniform(n, seed, -0.3, 0.9)
        assert np.array_equal(out.get(), ref)
        hip.random_normal(0, out.ptr, n, seed, 0.0, 1.0)
        got, ref = out.get(), hash_rng.random_normal(n, seed, 0.0, 1.0)
        ok = np.isfinite(ref)
        assert np.array_equal(np.isfinite(got), ok)
        assert np.abs(got[ok] - ref[ok]).max() <= 2e-6 * max(1.0, np.abs(ref[ok]).max())
        hip.random_normal(0, out.ptr, n, seed, -2.0, 0.01)
        got, ref = out.get(), hash_rng.random_normal(n, seed, -2.0, 0.01)
        assert np.abs(got[ok] - ref[ok]).max() <= 5e-7
    # a guard element after the end stays untouched
    g = DevArr(hip, np.full(130, 7.0, np.float32))
    hip.random_uniform(0, g.ptr, 129, 5, 0.0, 1.0)
    assert g.get()[129] == 7.0
    hip.random_normal(0, g.ptr, 0, 5, 0.0, 1.0)       # n = 0 is a no-op


def test_conv_descriptor_errors(hip):
    A = DevArr(hip, shape=(64,), fill=0.0)
    bad = hip.conv_desc(1, 1, 4, 4, 1, 3, 3, 4, 4, 1, 1, 0, 1)          # stride 0
    with pytest.raises(hip.HipException) as e:
        hip.conv2d_fwd(0, bad, A.ptr, A.ptr, A.ptr, 0)
    assert e.value.code == hip.ERR_INVALID
    big = hip.conv_desc(4096, 4096, 64, 64, 1, 3, 3, 64, 64, 1, 1, 1, 1)  # 256 GiB input
    with pytest.raises(hip.HipException) as e:
        hip.conv2d_fwd(0, big, A.ptr, A.ptr, A.ptr, 0)
    assert e.value.code == hip.ERR_UNSUPPORTED


# ------------------------------------------------------------------ unfold / transpose
def test_unfold_index_maps_bit_exact(hip):
    """Input element i holds the value i+1 (exact in fp32 up to 2^24), so the
    unfolded matrix reveals which flat input index every output element read."""
    for padding, d, s, ks in itertools.product(['same', 'valid', 2], [1, 2], [1, 2, 3], [5, 3, 2, 1]):
        n, c, o, h, w_ = 2, 3, 2, 9, 8
        if padding == 'valid' and min(h, w_) < (ks - 1) * d + 1:
            continue
        ci = info_conv2d(h, w_, ks, ks, s, d, padding)
        x = np.arange(1, n * c * h * w_ + 1, dtype=np.float32)
        X = DevArr(hip, x)
        for order, name in ((0, 'CJI_NHW'), (1, 'NHW_CJI')):
            shape, m = unfold_index_map(n, c, h, w_, ci.OH, ci.OW, ks, ks, ci.PADL, ci.PADT, d, s, name)
            out = DevArr(hip, shape=shape, fill=np.nan)
            hip.unfold2d(0, n, c, h, w_, ci.OH, ci.OW, ks, ks, ci.PADL, ci.PADT, d, s, order, False, X.ptr, out.ptr)
            assert np.array_equal(out.get().reshape(-1).astype(np.int64) - 1, m)
        dy = np.arange(1, n * o * ci.OH * ci.OW + 1, dtype=np.float32)
        DY = DevArr(hip, dy)
        shape, m = unfold_T_index_map(n, o, ci.OH, ci.OW, h, w_, ks, ks, ci.PADL, ci.PADT, d, s)
        out = DevArr(hip, shape=shape, fill=np.nan)
        hip.unfold2d(0, n, o, ci.OH, ci.OW, h, w_, ks, ks, ci.PADL, ci.PADT, d, s, 1, True, DY.ptr, out.ptr)
        assert np.array_equal(out.get().reshape(-1).astype(np.int64) - 1, m)


def test_transpose_exact(hip):
    rs = np.random.RandomState(1)
    for rank in (2, 3, 4, 5):
        for _ in range(4):
            shape = tuple(int(v) for v in rs.randint(1, 9, size=rank))
            axes = tuple(int(v) for v in rs.permutation(rank))
            v = rs.randint(256, size=shape).astype(np.float32)
            V = DevArr(hip, v)
            out = DevArr(hip, shape=tuple(shape[a] for a in axes), fill=1.0)
            hip.transpose(0, shape, axes, V.ptr, out.ptr, 1)
            assert np.array_equal(out.get() - 1.0, v.transpose(axes))


# ------------------------------------------------------------------ full-size properties
def _dot(a, b):
    return float(np.dot(a.astype(np.float64).ravel(), b.astype(np.float64).ravel()))


@pytest.mark.parametrize('xs,ws,s,d,padding', [((32, 128, 56, 56), (128, 128, 3, 3), 1, 1, 'same'),
                                               ((64, 256, 28, 28), (512, 256, 1, 1), 1, 1, 'valid'),
                                               ((16, 128, 32, 32), (256, 128, 5, 5), 2, 1, 2),
                                               ((32, 3, 224, 224), (64, 3, 7, 7), 2, 1, 3),
                                               ((16, 64, 64, 64), (64, 64, 3, 3), 1, 2, 2)])
def test_conv_full_size_adjoint_and_linearity(hip, xs, ws, s, d, padding):
    """At the benchmark sizes the oracle is too slow to run, but the three
    passes are tied together by identities that hold for any size:
      <conv(X, W), dY> = <X, dgrad(dY, W)> = <W, wgrad(X, dY)>        (adjoints)
      conv(X, W1 + W2) = conv(X, W1) + conv(X, W2)                    (linearity)
    and a dropped tap, a transposed operand or a wrong pad would break them.
    Sums are taken in fp64 on the host; tolerance 1e-5 of the magnitude sum."""
    rs = np.random.RandomState(77)
    desc, ci = _desc(hip, xs, ws, s, d, padding)
    x = rs.uniform(-1, 1, xs).astype(np.float32)
    w = rs.normal(0, 0.05, ws).astype(np.float32)
    w2 = rs.normal(0, 0.05, ws).astype(np.float32)
    dy = rs.normal(0, 1, (xs[0], ws[0], ci.OH, ci.OW)).astype(np.float32)
    say(f'full-size identities x={xs} w={ws}')
    if xs[1] == 3 and hip.device_info(0)['compute_units'] == 256:
        # the image stem at full batch takes the 16-row MFMA data gradient over a dY patch in LDS
        assert hip.conv2d_dgrad_path(desc, 0, 256)[0] == hip.DGRAD_PATH_STEM_MFMA
    X, W, W2, dY = DevArr(hip, x), DevArr(hip, w), DevArr(hip, w2), DevArr(hip, dy)
    Y, Y2, Y12 = (DevArr(hip, shape=dy.shape, fill=np.nan) for _ in range(3))
    dX, dW = DevArr(hip, shape=xs, fill=np.nan), DevArr(hip, shape=ws, fill=np.nan)
    hip.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, 0)
    hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, 0)
    hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, 0)
    y, dx, dw = Y.get(), dX.get(), dW.get()
    a, b, c = _dot(y, dy), _dot(x, dx), _dot(w, dw)
    scale = float(np.dot(np.abs(y).astype(np.float64).ravel(), np.abs(dy).astype(np.float64).ravel()))
    assert abs(a - b) <= 1e-5 * scale and abs(a - c) <= 1e-5 * scale, (a, b, c, scale)
    W12 = DevArr(hip, w + w2)
    hip.conv2d_fwd(0, desc, X.ptr, W2.ptr, Y2.ptr, 0)
    hip.conv2d_fwd(0, desc, X.ptr, W12.ptr, Y12.ptr, 0)
    assert rel_err(Y12.get(), y.astype(np.float64) + Y2.get()) <= 1e-5
    # accumulation: a second '+=' pass doubles a gradient exactly
    hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, 1)
    assert np.array_equal(dW.get(), dw + dw)


def test_gemm_full_size_adjoints(hip):
    """<A.B, dC> = <A, dC.B^T> = <B, A^T.dC> at 4096^3."""
    rs = np.random.RandomState(78)
    n = 4096
    a, b, dc = (rs.normal(0, 1, (n, n)).astype(np.float32) for _ in range(3))
    A, B, D = DevArr(hip, a), DevArr(hip, b), DevArr(hip, dc)
    C, dA, dB = (DevArr(hip, shape=(n, n), fill=np.nan) for _ in range(3))
    say('gemm 4096^3 adjoint identities')
    hip.gemm(0, 0, 0, 1, n, n, n, A.ptr, n, 0, B.ptr, n, 0, C.ptr, n, 0, 0)
    hip.gemm(0, 0, 1, 1, n, n, n, D.ptr, n, 0, B.ptr, n, 0, dA.ptr, n, 0, 0)
    hip.gemm(0, 1, 0, 1, n, n, n, A.ptr, n, 0, D.ptr, n, 0, dB.ptr, n, 0, 0)
    c = C.get()
    x, y, z = _dot(c, dc), _dot(a, dA.get()), _dot(b, dB.get())
    scale = float(np.dot(np.abs(c).astype(np.float64).ravel(), np.abs(dc).astype(np.float64).ravel()))
    assert abs(x - y) <= 1e-5 * scale and abs(x - z) <= 1e-5 * scale, (x, y, z, scale)
    rows = np.arange(0, n, 511)
    assert rel_err(c[rows], a[rows].astype(np.float64) @ b.astype(np.float64)) <= TOL

