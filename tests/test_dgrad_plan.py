"""Host-side plan of the data gradient (lnn_conv2d_dgrad_path: no device needed).  For every geometry the
vector-ALU kernel accepts, the dY tile one block brings to LDS must fit the kernel's LDS plane and every window a
thread reads must lie inside the rows / columns that were brought in; the selection between the kernel families
must follow the documented rules, whatever the compute-unit count of the device."""
import itertools

from litenn_amd.core.hip import api
from oracle import info_conv2d

SUPPORTED = {1: (1, 3, 5), 2: (3, 4, 5, 7)}


def _desc(N, C, H, W, O, K, s, d, padding):
    ci = info_conv2d(H, W, K, K, s, d, padding)
    return api.conv_desc(N, C, H, W, O, K, K, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)


def test_vector_path_tiles_stay_inside_their_lds_plane():
    n_vec = 0
    for s, ks in SUPPORTED.items():
        for K in ks:
            pads = ['same', 'valid'] + list(range(0, K + 1)) + [(0, K, 1, 0), (K, 0, 0, 2), (1, 2, 3, 0)]
            for padding, (H, W), C, beta in itertools.product(pads, [(70, 66), (64, 64), (33, 97), (224, 224)],
                                                               [1, 3, 4], [0, 1]):
                if padding == 'valid' and min(H, W) < K:
                    continue
                path, t = api.conv2d_dgrad_path(_desc(512, C, H, W, 8, K, s, 1, padding), beta, 256)
                # every supported (S, K) has taps in every pixel class, so nothing falls back at this batch size
                assert path == api.DGRAD_PATH_VECTOR, (s, K, padding, H, W, C, beta)
                n_vec += 1
                tag = (s, K, padding, H, W, C, beta, t)
                assert 0 < t['rows'] <= t['max_extent'] and 0 < t['cols'] <= t['max_extent'], tag
                assert t['max_extent'] == 16 + (K + s - 1) // s + 1, tag
                assert t['min_row'] >= 0 and t['min_col'] >= 0, tag
                assert t['max_row'] < t['rows'] and t['max_col'] < t['cols'], tag
    assert n_vec > 1000


def test_selection_rules():
    big = dict(N=64, H=70, W=66, O=16)

    def path(C, K, s, d=1, padding='same', N=big['N'], cus=256, beta=1, O=big['O']):
        return api.conv2d_dgrad_path(_desc(N, C, big['H'], big['W'], O, K, s, d, padding), beta, cus)[0]

    assert path(3, 7, 2, padding=3) == api.DGRAD_PATH_VECTOR
    assert path(4, 3, 1) == api.DGRAD_PATH_VECTOR
    assert path(5, 3, 1) == api.DGRAD_PATH_MFMA_TABLE             # more than four channels
    assert path(3, 3, 1, d=2) == api.DGRAD_PATH_MFMA_TABLE        # dilation
    assert path(3, 5, 3, padding=2) == api.DGRAD_PATH_MFMA_TABLE  # stride 3
    assert path(3, 7, 1) == api.DGRAD_PATH_MFMA_TABLE             # 7 x 7 at stride 1
    assert path(3, 3, 1, O=32) == api.DGRAD_PATH_VECTOR           # C decides, not O
    assert path(8, 3, 1, O=32) == api.DGRAD_PATH_MFMA_TAP
    # too few tiles for the chip: 5 x 5 tiles of 16 x 16 per 70 x 66 image at stride 1, one block each
    assert path(3, 3, 1, N=10, cus=256) == api.DGRAD_PATH_MFMA_TABLE       # 250 blocks < 256
    assert path(3, 3, 1, N=11, cus=256) == api.DGRAD_PATH_VECTOR           # 275 blocks
    assert path(3, 3, 1, N=10, cus=128) == api.DGRAD_PATH_VECTOR           # the same problem on a smaller part
    assert path(3, 3, 1, N=1, cus=304) == api.DGRAD_PATH_MFMA_TABLE


def test_stem_mfma_selection():
    """LNN_DGRAD_PATH_STEM_MFMA: stride 2, no dilation, at most four input channels, 32 or more output channels in
    multiples of 8, at most four dY rows and columns per pair of input pixels, two tiles of 32 x 32 pixels per compute
    unit; everything else keeps its earlier path."""
    def path(C=3, O=64, K=7, s=2, d=1, padding=3, N=32, H=224, cus=256):
        return api.conv2d_dgrad_path(_desc(N, C, H, H, O, K, s, d, padding), 0, cus)[0]

    assert path() == api.DGRAD_PATH_STEM_MFMA
    for kw in (dict(C=4), dict(C=1), dict(O=32), dict(O=72), dict(K=5, padding=2), dict(K=3, padding=1), dict(K=2, padding=0),
               dict(K=7, padding='valid'), dict(K=8, padding=2), dict(K=4, padding=1)):
        assert path(**kw) == api.DGRAD_PATH_STEM_MFMA, kw
    for kw in (dict(C=5), dict(O=24), dict(O=36), dict(s=1, K=3, padding=1), dict(d=2), dict(K=9, padding=4), dict(K=8, padding=3),
               dict(s=3, K=5, padding=2)):
        assert path(**kw) != api.DGRAD_PATH_STEM_MFMA, kw
    # 224 x 224 pixels = 49 tiles per image: 512 tiles from 11 images on 256 compute units
    assert path(N=11) == api.DGRAD_PATH_STEM_MFMA and path(N=10) == api.DGRAD_PATH_VECTOR
    assert path(N=10, cus=240) == api.DGRAD_PATH_STEM_MFMA


def test_bad_arguments():
    import pytest
    d = _desc(4, 3, 16, 16, 4, 3, 1, 1, 'same')
    with pytest.raises(api.HipException) as e:
        api.conv2d_dgrad_path(d, 0, 0)
    assert e.value.code == api.ERR_INVALID
    bad = api.conv_desc(1, 1, 4, 4, 1, 3, 3, 4, 4, 1, 1, 0, 1)
    with pytest.raises(api.HipException):
        api.conv2d_dgrad_path(bad, 0, 256)


def test_forward_path_selection():
    """lnn_conv2d_fwd_path: the patch kernels take three input channels, 33-64 output channels, square 3x3
    (stride 1 or 2), 5x5 and 7x7 (stride 2) kernels without dilation, from four 256-pixel tiles per compute unit."""
    import pytest

    def path(C=3, O=64, K=7, s=2, d=1, N=32, H=224, cus=256, KW=None):
        KW = K if KW is None else KW
        ci = info_conv2d(H, H, K, KW, s, d, 'same')
        return api.conv2d_fwd_path(api.conv_desc(N, C, H, H, O, K, KW, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d), cus)

    assert path() == api.FWD_PATH_STEM_PATCH
    for k, s in ((3, 1), (3, 2), (5, 2), (7, 2)):
        assert path(K=k, s=s) == api.FWD_PATH_STEM_PATCH
        assert path(K=k, s=s, O=33) == api.FWD_PATH_STEM_PATCH
    for kw in (dict(C=4), dict(C=1), dict(O=32), dict(O=65), dict(K=5, s=1), dict(K=7, s=1), dict(K=3, s=3), dict(d=2),
               dict(K=3, KW=5, s=1), dict(K=9)):
        assert path(**kw) == api.FWD_PATH_IMPLICIT_GEMM, kw
    # 112 x 112 output pixels = 49 tiles per image: 1024 tiles from 21 images on 256 compute units
    assert path(N=21) == api.FWD_PATH_STEM_PATCH and path(N=20) == api.FWD_PATH_IMPLICIT_GEMM
    assert path(N=20, cus=240) == api.FWD_PATH_STEM_PATCH
    with pytest.raises(api.HipException) as e:
        path(cus=0)
    assert e.value.code == api.ERR_INVALID
