"""Seeded random-geometry differential test of the three convolution passes on the GPU against the fp64 oracle.

The kernels choose among many code paths by geometry (channel counts that fill or do not fill the 32-wide K step,
C <= 4, image stems, pixel classes of a strided data gradient, K splits and remainder cuts that depend on how the tile
count compares with the number of compute units).  Hand-picked grids pin each path; this test draws geometries at random,
biased towards the values where the plans flip, so that combinations nobody listed get exercised too.  Integer-valued
data, exact equality (every partial sum is representable, so the order of summation cannot show), '=' into NaN-filled
outputs and '+=' into prefilled ones, the plain entry points and - where lnn_conv2d_weights_plan allows - the ones that
take the permuted weight copy.  Stops at the first failure and names the geometry.
"""
import numpy as np
import pytest

from oracle import conv2d_dw, conv2d_dx, conv2d_fwd, info_conv2d
from tests.gpu_util import DevArr, say

pytestmark = pytest.mark.gpu

CHANNELS = [1, 2, 3, 4, 5, 8, 12, 16, 31, 32, 33, 36, 48, 64, 65, 96, 128, 160]


def _draw(rs, max_macs):
    """One geometry whose forward pass costs at most max_macs multiply-adds."""
    while True:
        kh = int(rs.choice([1, 2, 3, 3, 4, 5, 5, 7]))
        kw = kh if rs.rand() < 0.7 else int(rs.choice([1, 2, 3, 4, 5, 7]))
        s = int(rs.choice([1, 1, 2, 2, 3]))
        d = int(rs.choice([1, 1, 1, 2]))
        c, o = int(rs.choice(CHANNELS)), int(rs.choice(CHANNELS))
        n = int(rs.choice([1, 1, 2, 3, 5, 8]))
        ih, iw = int(rs.randint(1, 26)), int(rs.randint(1, 26))
        kind = rs.randint(5)
        if kind == 0:
            padding = 'same'
        elif kind == 1:
            padding = 'valid'
        elif kind == 2:
            padding = int(rs.randint(0, 4))
        else:
            padding = tuple(int(v) for v in rs.randint(0, 4, size=4))
        ekh, ekw = (kh - 1) * d + 1, (kw - 1) * d + 1
        if padding == 'valid' and (ih < ekh or iw < ekw):
            continue
        ci = info_conv2d(ih, iw, kh, kw, s, d, padding)
        if n * o * ci.OH * ci.OW * c * kh * kw > max_macs:
            continue
        return (n, c, ih, iw), (o, c, kh, kw), s, d, padding, ci


def _check_case(hip, rs, xs, ws, s, d, padding, ci, images=None, tag=''):
    """All three passes of one geometry, '=' and '+=', plain and permuted-weight entry points.  images: which images of
    the batch go to the oracle for Y and dX (None: all); dW always needs, and gets, the whole batch."""
    n, c, ih, iw = xs
    o, _, kh, kw = ws
    desc = hip.conv_desc(n, c, ih, iw, o, kh, kw, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)
    where = f'{tag}x={xs} w={ws} stride={s} dilation={d} padding={padding!r}'
    say('random geometry ' + where)
    # values small enough that every sum stays below 2**24
    hi_x = 16 if c * kh * kw * 225 < (1 << 23) else 4
    x = rs.randint(hi_x, size=xs).astype(np.float32)
    w = (rs.randint(hi_x, size=ws) - hi_x // 4).astype(np.float32)
    hi_y = 8 if n * ci.OH * ci.OW * 15 * 7 < (1 << 23) else 2
    dy = (rs.randint(hi_y, size=(n, o, ci.OH, ci.OW)) - hi_y // 4).astype(np.float32)
    X, W, dY = DevArr(hip, x), DevArr(hip, w), DevArr(hip, dy)
    imgs = list(range(n)) if images is None else sorted(set(images))
    ry = {i: conv2d_fwd(x[i:i + 1], w, s, d, padding)[0] for i in imgs}
    rdx = {i: conv2d_dx(dy[i:i + 1], w, (1,) + xs[1:], s, d, padding)[0] for i in imgs}
    rdw = np.zeros(ws, np.float64)
    for i0 in range(0, n, 8):
        rdw += conv2d_dw(x[i0:i0 + 8], dy[i0:i0 + 8], ws, s, d, padding)
    fwd_pw, dx_pw = hip.conv2d_weights_plan(desc, hip.PASS_FWD), hip.conv2d_weights_plan(desc, hip.PASS_DGRAD)
    Wp = None
    if fwd_pw or dx_pw:
        Wp = DevArr(hip, shape=(o, kh * kw, c), fill=np.nan)
        hip.conv2d_permute_weights(0, desc, W.ptr, hip.W_OIHW, Wp.ptr)
    y0 = rs.randint(-3, 4, size=dy.shape).astype(np.float32)
    x0 = rs.randint(-3, 4, size=xs).astype(np.float32)
    w0 = rs.randint(-3, 4, size=ws).astype(np.float32)
    for beta in (0, 1):
        for use_wp in ((False, True) if Wp is not None else (False,)):
            Y = DevArr(hip, y0) if beta else DevArr(hip, shape=dy.shape, fill=np.nan)
            if use_wp and fwd_pw:
                hip.conv2d_fwd_pw(0, desc, X.ptr, Wp.ptr, None, hip.ACT_NONE, 0.0, Y.ptr, beta)
            else:
                hip.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, beta)
            got = Y.get()
            for i in imgs:
                assert np.array_equal(got[i], ry[i] + (y0[i] if beta else 0)), f'forward beta={beta} wp={use_wp} image {i}: {where}'
            dX = DevArr(hip, x0) if beta else DevArr(hip, shape=xs, fill=np.nan)
            if use_wp and dx_pw:
                hip.conv2d_dgrad_pw(0, desc, dY.ptr, Wp.ptr, dX.ptr, beta)
            else:
                hip.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, beta)
            got = dX.get()
            for i in imgs:
                assert np.array_equal(got[i], rdx[i] + (x0[i] if beta else 0)), f'dgrad beta={beta} wp={use_wp} image {i}: {where}'
            if images is not None:   # the images that did not go to the oracle must at least have been written
                assert np.isfinite(got).all(), f'dgrad left elements unwritten: {where}'
        dW = DevArr(hip, w0) if beta else DevArr(hip, shape=ws, fill=np.nan)
        hip.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, beta)
        assert np.array_equal(dW.get(), rdw + (w0 if beta else 0)), f'wgrad beta={beta}: {where}'


def test_random_small_geometries_integer_exact(hip):
    rs = np.random.RandomState(20240)
    for k in range(300):
        xs, ws, s, d, padding, ci = _draw(rs, 3_000_000)
        _check_case(hip, rs, xs, ws, s, d, padding, ci, tag=f'#{k} ')


def _n_for_tiles(tiles_per_image, target):
    return max(1, -(-target // tiles_per_image))


def test_geometries_at_the_plan_boundaries_integer_exact(hip):
    """Shapes just below, at and just above the gates that compare a tile count with the number of compute units: the
    image-stem kernels (4 tiles of 256 output pixels per compute unit forward / weight gradient, 2 tiles of 32 x 32 input
    pixels data gradient), the paired pixel classes of a strided data gradient with 33-64 input channels, and the K split
    / remainder cut of forward and data gradient (output units against 1x and 5x the compute units).  The first, a middle
    and the last image of every batch go to the oracle."""
    rs = np.random.RandomState(20241)
    cus = hip.device_info(0)['compute_units']
    cases, stem_fwd, stem_dgrad = [], {}, {}
    # stem forward / weight gradient: C = 3, O in 33..64
    for (k, s, o, oh, ow) in ((3, 1, 40, 48, 48), (3, 2, 33, 40, 52), (5, 2, 64, 32, 36), (7, 2, 48, 30, 34)):
        tiles = (oh * ow + 255) // 256
        for dn in (-1, 0, 1):
            n = _n_for_tiles(tiles, 4 * cus) + dn
            cases.append(((n, 3, oh * s, ow * s), (o, 3, k, k), s, 1, 'same'))
            stem_fwd[len(cases) - 1] = dn >= 0
    # stem data gradient: C <= 4, stride 2, O % 8 == 0 from 32
    for (c, o, k, ih, iw) in ((3, 32, 5, 66, 62), (4, 40, 3, 64, 64), (1, 64, 7, 33, 95)):
        tiles = (((ih + 1) // 2 + 15) // 16) * (((iw + 1) // 2 + 15) // 16)
        for dn in (-1, 0, 1):
            n = _n_for_tiles(tiles, 2 * cus) + dn
            cases.append(((n, c, ih, iw), (o, c, k, k), 2, 1, 'same'))
            stem_dgrad[len(cases) - 1] = dn >= 0
    # paired pixel classes: 33..64 input channels, O % 32 == 0, stride 2, class planes of 2 * cus sub-tiles of 128 columns
    for (c, o, k, hw) in ((64, 32, 3, 32), (48, 64, 5, 24), (36, 32, 3, 40)):
        per_img = (hw // 2) * (hw // 2)
        n0 = -(-(cus // 4 * 2 * 2 * 64) // per_img)
        for dn in (-1, 0, 1):
            cases.append(((n0 + dn, c, hw, hw), (o, c, k, k), 2, 1, 'same'))
    # forward / data gradient with the output units around 1x and 5x the compute units (K split, remainder cut)
    for (c, o, k, s, hw, mult) in ((64, 32, 3, 1, 32, 1), (32, 128, 5, 1, 16, 1), (64, 64, 3, 2, 48, 1), (32, 32, 3, 1, 40, 5),
                                   (96, 160, 3, 1, 12, 1)):
        unit = 32 if o > 64 else (64 if o > 32 else 128)
        m_tiles = -(-o // (32 if o <= 32 else (64 if o <= 64 else 128)))
        oh = -(-hw // s)
        per_img = oh * oh
        n0 = max(1, (mult * cus * unit) // (per_img * m_tiles))
        for dn in (0, 1):
            cases.append(((n0 + dn, c, hw, hw), (o, c, k, k), s, 1, 'same'))
    for j, (xs, ws, s, d, padding) in enumerate(cases):
        ci = info_conv2d(xs[2], xs[3], ws[2], ws[3], s, d, padding)
        n = xs[0]
        desc = hip.conv_desc(n, xs[1], xs[2], xs[3], ws[0], ws[2], ws[3], ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)
        if j in stem_fwd:      # the gate sits where this test thinks it does
            assert (hip.conv2d_fwd_path(desc, cus) == hip.FWD_PATH_STEM_PATCH) == stem_fwd[j], (xs, ws)
        if j in stem_dgrad:
            assert (hip.conv2d_dgrad_path(desc, 0, cus)[0] == hip.DGRAD_PATH_STEM_MFMA) == stem_dgrad[j], (xs, ws)
        _check_case(hip, rs, xs, ws, s, d, padding, ci, images=(0, n // 2, n - 1), tag=f'gate #{j} ')
