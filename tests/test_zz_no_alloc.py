"""The allocation-free entry point lnn_conv2d_wgrad_noalloc_f32 against lnn_conv2d_wgrad_f32 through the C ABI.

Both run the same kernels with the same plan, so the results must agree bit for bit on float data too: '=' and '+=',
the pixel-major kernels with split-K partial sums, the table-driven kernel (gather table carved from the fixed
scratch array), and a problem without any K split.  Two calls in a row, the second on a smaller input, pin that
nothing of the first call's scratch contents leaks into the second.  A problem whose scratch exceeds the array
is rejected with UNSUPPORTED and leaves the output untouched."""
import numpy as np
import pytest

from oracle import conv2d_dw, info_conv2d
from tests.gpu_util import DevArr, say

pytestmark = pytest.mark.gpu


def _case(hip, xs, ws, s, d, padding, seed, integer=False):
    rs = np.random.RandomState(seed)
    ci = info_conv2d(xs[2], xs[3], ws[2], ws[3], s, d, padding)
    desc = hip.conv_desc(xs[0], xs[1], xs[2], xs[3], ws[0], ws[2], ws[3], ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)
    ys = (xs[0], ws[0], ci.OH, ci.OW)
    if integer:
        x, dy = rs.randint(-4, 5, size=xs).astype(np.float32), rs.randint(-4, 5, size=ys).astype(np.float32)
    else:
        x, dy = rs.uniform(-1, 1, xs).astype(np.float32), rs.normal(0, 1, ys).astype(np.float32)
    return desc, x, dy


def _both(hip, xs, ws, s, d, padding, seed, integer=False):
    desc, x, dy = _case(hip, xs, ws, s, d, padding, seed, integer)
    X, dY = DevArr(hip, x), DevArr(hip, dy)
    out = {}
    for beta, fill in ((0, np.nan), (1, 0.5)):
        ref, got = DevArr(hip, shape=ws, fill=fill), DevArr(hip, shape=ws, fill=fill)
        hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, ref.ptr, beta)
        hip.conv2d_wgrad_noalloc(0, desc, X.ptr, dY.ptr, got.ptr, beta)
        r, g = ref.get(), got.get()
        assert np.array_equal(r, g), (xs, ws, s, d, padding, beta)
        assert np.isfinite(g).all()
        out[beta] = g
    return x, dy, out


def test_noalloc_wgrad_matches_the_allocating_entry_point_twice_in_a_row(hip):
    # first call: the benchmark layer at reduced batch (pixel-major kernel, ~50 K slices of partial sums)
    big = ((8, 128, 56, 56), (128, 128, 3, 3), 1, 1, 'same')
    say(f'noalloc wgrad {big}')
    _both(hip, *big, seed=1)
    # second call, smaller: fewer slices, so most of the array still holds the first call's partial sums
    small = ((2, 64, 12, 12), (40, 64, 3, 3), 1, 1, 'same')
    say(f'noalloc wgrad {small}')
    x, dy, out = _both(hip, *small, seed=2, integer=True)
    assert np.array_equal(out[0], conv2d_dw(x, dy, small[1], 1, 1, 'same'))     # and exact against the oracle
    # table-driven kernel: the gather table lives at the tail of the same array
    stem = ((4, 3, 40, 40), (24, 3, 7, 7), 2, 1, 3)
    say(f'noalloc wgrad {stem}')
    x, dy, out = _both(hip, *stem, seed=3, integer=True)
    assert np.array_equal(out[0], conv2d_dw(x, dy, stem[1], 2, 1, 3))
    # strided, 128-bit pixel gather, many output channels, no K split needed
    for case in (((2, 32, 20, 20), (130, 32, 5, 5), 2, 1, 2), ((4, 256, 28, 28), (512, 256, 1, 1), 1, 1, 'valid'),
                 ((1, 1024, 8, 8), (1024, 1024, 3, 3), 1, 1, 'same')):
        say(f'noalloc wgrad {case}')
        _both(hip, *case, seed=4)
    # an image stem at a batch that takes the patch kernel: its blocks' partial results (10 MiB) live in the same array
    patch = ((24, 3, 224, 224), (64, 3, 7, 7), 2, 1, 3)
    say(f'noalloc wgrad {patch}')
    _both(hip, *patch, seed=7)
    # and the first, large shape again after the small ones
    _both(hip, *big, seed=5)


def test_noalloc_wgrad_rejects_what_does_not_fit(hip):
    """One output tile (O = 128, C*KH*KW = 256) and a long K: 256 slices of 128 x 256 partial sums fill the 32 MiB
    array exactly.  Output planes of 5 x 5 pixels are too small for the kernels that need no table, and the
    table-driven kernel's gather table no longer fits behind the partial sums."""
    if hip.device_info(0)['compute_units'] != 256:
        pytest.skip('the shape is laid out for 256 compute units')
    xs, ws = (1311, 8, 8, 12), (128, 8, 4, 8)
    desc, x, dy = _case(hip, xs, ws, 1, 1, 'valid', 6)
    X, dY = DevArr(hip, x), DevArr(hip, dy)
    dW = DevArr(hip, shape=ws, fill=7.0)
    say('noalloc wgrad over the scratch limit')
    with pytest.raises(hip.HipException) as e:
        hip.conv2d_wgrad_noalloc(0, desc, X.ptr, dY.ptr, dW.ptr, 1)
    assert e.value.code == hip.ERR_UNSUPPORTED and 'scratch' in e.value.message
    assert np.all(dW.get() == 7.0)
    ref = DevArr(hip, shape=ws, fill=7.0)
    hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, ref.ptr, 1)                         # the allocating entry point takes it
    assert np.isfinite(ref.get()).all() and not np.all(ref.get() == 7.0)
