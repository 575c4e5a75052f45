"""GPU parity of the GEMM kernel families behind nn.matmul / nn.Dense (matmul.py:33-72, module/Dense.py:44-48,
spatial_affine_transform2D.py:33-36): the wavefront-tile kernel for few rows or a short K, the tile engine cut along
K for few output tiles, and the row-per-thread kernel for K and N of a handful.  Bit-exact on integer-valued data
against numpy (every partial sum is exactly representable, so the order of summation cannot show), 1e-4 normalised
against fp64 on float data."""
import numpy as np
import pytest

from tests.gpu_util import DevArr, rel_err, say

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _operands(rs, ta, tb, batch, M, N, K, pad_rows, lda=None, ldb=None):
    """Integer-valued operands.  Each batch item is followed by pad_rows rows of NaN: a kernel that relies on rows
    past K reading as zeros must get them from the range check, not from memory."""
    a_rows, a_cols = (K, M) if ta else (M, K)
    b_rows, b_cols = (N, K) if tb else (K, N)
    lda, ldb = lda or a_cols, ldb or b_cols
    a = np.full((batch, a_rows + pad_rows, lda), np.nan, np.float32)
    b = np.full((batch, b_rows + pad_rows, ldb), np.nan, np.float32)
    a[:, :a_rows, :a_cols] = rs.randint(16, size=(batch, a_rows, a_cols))
    b[:, :b_rows, :b_cols] = rs.randint(16, size=(batch, b_rows, b_cols))
    av, bv = a[:, :a_rows, :a_cols].astype(np.float64), b[:, :b_rows, :b_cols].astype(np.float64)
    ref = np.matmul(av.transpose(0, 2, 1) if ta else av, bv.transpose(0, 2, 1) if tb else bv)
    return a, b, ref


def _check(hip, rs, ta, tb, batch, M, N, K, pad_rows=3, lda=None, ldb=None, with_bias=True):
    a, b, ref = _operands(rs, ta, tb, batch, M, N, K, pad_rows, lda, ldb)
    c0 = rs.randint(8, size=(batch, M, N)).astype(np.float32)
    A, B = DevArr(hip, a), DevArr(hip, b)
    sa, sb = a.shape[1] * a.shape[2], b.shape[1] * b.shape[2]
    for beta in (0, 1):
        say(f'gemm ta={ta} tb={tb} batch={batch} M={M} N={N} K={K} lda={a.shape[2]} ldb={b.shape[2]} beta={beta}')
        C = DevArr(hip, c0)
        hip.gemm(0, ta, tb, batch, M, N, K, A.ptr, a.shape[2], sa, B.ptr, b.shape[2], sb, C.ptr, N, M * N, beta)
        assert np.array_equal(C.get(), ref + (c0 if beta else 0)), (ta, tb, batch, M, N, K, beta)
    if with_bias:
        bias = (rs.randint(-8, 8, size=N) - ref[0, 0, :]).astype(np.float32)   # row 0 lands around zero: both signs occur
        Bi = DevArr(hip, bias)
        for act, slope in ((hip.ACT_NONE, 0.0), (hip.ACT_LEAKY_RELU, 0.25)):
            say(f'gemm_bias_act ta={ta} tb={tb} batch={batch} M={M} N={N} K={K} act={act}')
            C = DevArr(hip, shape=(batch, M, N), fill=np.nan)
            hip.gemm_bias_act(0, ta, tb, batch, M, N, K, A.ptr, a.shape[2], sa, B.ptr, b.shape[2], sb, Bi.ptr, act, slope,
                              C.ptr, N, M * N)
            want = (ref + bias.astype(np.float64)).astype(np.float32)
            if act:
                want = np.where(want >= 0, want, np.float32(slope) * want)
            assert np.array_equal(C.get(), want), (ta, tb, batch, M, N, K, act)
            assert N < 8 or ((want < 0).any() and (want > 0).any())


@pytest.mark.parametrize('M', [1, 7, 32, 33, 64])
def test_dense_forward_few_rows(hip, M):
    """x[M, in] . w[in, out]: the weight matrix streamed once (wavefront tiles, K split inside and across workgroups)."""
    rs = np.random.RandomState(100 + M)
    for N, K in ((512, 4096), (384, 1024), (132, 8192), (4096, 512), (128, 64), (1024, 200)):
        _check(hip, rs, 0, 0, 1, M, N, K)
    _check(hip, rs, 0, 0, 3, M, 256, 1024)                      # batched: no slices through memory
    _check(hip, rs, 0, 0, 1, M, 260, 2048, lda=2052, ldb=264)   # padded leading dimensions


@pytest.mark.parametrize('M', [1, 7, 32, 64])
def test_dense_data_gradient_few_rows(hip, M):
    """dy[M, out] . w[in, out]^T: few output tiles and a long K, cut along K on the tile engine."""
    rs = np.random.RandomState(200 + M)
    for N, K in ((512, 4096), (384, 1024), (130, 4100), (4096, 512)):
        _check(hip, rs, 0, 1, 1, M, N, K)


@pytest.mark.parametrize('K', [1, 7, 32, 33, 64])
def test_dense_weight_gradient_short_k(hip, K):
    """x[K, in]^T . dy[K, out]: the result streamed once (wavefront tiles, no K split, '+=' prefetched)."""
    rs = np.random.RandomState(300 + K)
    for M, N in ((512, 512), (1000, 260), (96, 4096), (4096, 128)):
        _check(hip, rs, 1, 0, 1, M, N, K, with_bias=(M == 512))
    _check(hip, rs, 1, 0, 2, 300, 256, K, with_bias=False)
    _check(hip, rs, 1, 0, 1, 260, 256, K, lda=264, ldb=260, with_bias=False)


def test_few_tiles_long_k_all_layouts(hip):
    """More rows than the wavefront-tile kernel takes, still fewer tiles than compute units: engine with a K split,
    aligned (operands straight into LDS) and ragged (through registers)."""
    rs = np.random.RandomState(7)
    for ta, tb in ((0, 0), (0, 1), (1, 0)):
        for M, N, K in ((128, 256, 4096), (96, 512, 2048), (130, 200, 4100), (300, 36, 3001), (256, 1024, 1024)):
            _check(hip, rs, ta, tb, 1, M, N, K)


def test_small_k_small_n_rows(hip):
    """[N, H*W, 3] . [N, 3, 2] of a spatial transform and its data gradient [N, H*W, 2] . [N, 3, 2]^T."""
    rs = np.random.RandomState(11)
    for batch, M, N, K in ((5, 1000, 2, 3), (1, 256, 8, 8), (16, 4096, 2, 3), (2, 777, 1, 1), (3, 300, 5, 7)):
        _check(hip, rs, 0, 0, batch, M, N, K, pad_rows=0)
        _check(hip, rs, 0, 1, batch, M, N, K, pad_rows=0, with_bias=False)


def test_dense_float_tolerance(hip):
    rs = np.random.RandomState(0)
    B, I, O = 32, 4096, 4096
    x = rs.normal(0, 1, (B, I)).astype(np.float32)
    w = rs.normal(0, 1, (I, O)).astype(np.float32)
    dy = rs.normal(0, 1, (B, O)).astype(np.float32)
    bias = rs.normal(0, 1, O).astype(np.float32)
    X, W, dY, Bi = DevArr(hip, x), DevArr(hip, w), DevArr(hip, dy), DevArr(hip, bias)
    Y, dX, dW = DevArr(hip, shape=(B, O), fill=np.nan), DevArr(hip, shape=(B, I), fill=np.nan), DevArr(hip, shape=(I, O), fill=0.5)
    say('dense 32 x 4096 x 4096: forward with bias, dX, dW (+=)')
    hip.gemm_bias_act(0, 0, 0, 1, B, O, I, X.ptr, I, 0, W.ptr, O, 0, Bi.ptr, hip.ACT_NONE, 0.0, Y.ptr, O, 0)
    hip.gemm(0, 0, 1, 1, B, I, O, dY.ptr, O, 0, W.ptr, O, 0, dX.ptr, I, 0, 0)
    hip.gemm(0, 1, 0, 1, I, O, B, X.ptr, I, 0, dY.ptr, O, 0, dW.ptr, O, 0, 1)
    x64, w64, d64 = x.astype(np.float64), w.astype(np.float64), dy.astype(np.float64)
    assert rel_err(Y.get(), x64 @ w64 + bias) <= TOL
    assert rel_err(dX.get(), d64 @ w64.T) <= TOL
    assert rel_err(dW.get(), x64.T @ d64 + 0.5) <= TOL


def test_bias_act_bwd_rows_layout(hip):
    """Backward of the dense epilogue: planes of one element (y[rows][features])."""
    rs = np.random.RandomState(5)
    for rows, feats in ((32, 4096), (7, 100), (300, 33), (1, 5)):
        y = (rs.randint(9, size=(rows, feats)) - 4).astype(np.float32)
        dy = rs.randint(16, size=(rows, feats)).astype(np.float32)
        db0 = rs.randint(8, size=feats).astype(np.float32)
        Y, dY = DevArr(hip, y), DevArr(hip, dy)
        for beta in (0, 1):
            say(f'bias_act_bwd rows={rows} features={feats} beta={beta}')
            dP, dB = DevArr(hip, shape=(rows, feats), fill=np.nan), DevArr(hip, db0)
            hip.bias_act_bwd(0, rows, feats, 1, Y.ptr, dY.ptr, hip.ACT_LEAKY_RELU, 0.5, dP.ptr, dB.ptr, beta)
            pre = dy * np.where(y >= 0, 1.0, 0.5).astype(np.float32)
            assert np.array_equal(dP.get(), pre)
            assert np.array_equal(dB.get(), pre.sum(0) + (db0 if beta else 0))


def test_lr_dropout_updates_match_the_hash_oracle(hip):
    """lnn_*_update_multi_lrd_f32 against the oracle's counter hash, bit for bit: two tensors per launch, every seed
    position, with and without nesterov (Optimizer.py:186-203, SGD.py:42-74, Adam.py:61-72)."""
    from oracle import hash_rng
    rs = np.random.RandomState(9)
    ns = [70001, 333]
    p, lr, mom = 0.4, 0.5, 0.5
    w0 = [rs.randint(-8, 9, size=n).astype(np.float32) for n in ns]
    g = [rs.randint(1, 9, size=n).astype(np.float32) for n in ns]
    a0 = [rs.randint(-4, 5, size=n).astype(np.float32) for n in ns]
    seeds = [12345, 2147483647, 4294967295 - 100, 7]     # the third wraps the 32-bit counter inside the tensor
    for nesterov in (0, 1):
        say(f'sgd_update_multi_lrd nesterov={nesterov}')
        W, G, A = [DevArr(hip, x) for x in w0], [DevArr(hip, x) for x in g], [DevArr(hip, x) for x in a0]
        hip.sgd_update_multi_lrd(0, ns, [x.ptr for x in W], [x.ptr for x in G], [x.ptr for x in A], mom, lr, nesterov, p, seeds)
        for i, n in enumerate(ns):
            lr_a = np.where(hash_rng.lr_dropout_mask(n, seeds[2 * i], p), 0.0, lr)
            lr_t = np.where(hash_rng.lr_dropout_mask(n, seeds[2 * i + 1], p), 0.0, lr)
            acc = mom * a0[i].astype(np.float64) - lr_a * g[i]
            w = w0[i] + (mom * acc - lr_t * g[i] if nesterov else acc)
            assert np.array_equal(A[i].get(), acc) and np.array_equal(W[i].get(), w)
    say('adam_update_multi_lrd')
    W, G = [DevArr(hip, x) for x in w0], [DevArr(hip, x) for x in g]
    M, V = [DevArr(hip, np.zeros(n, np.float32)) for n in ns], [DevArr(hip, np.zeros(n, np.float32)) for n in ns]
    hip.adam_update_multi_lrd(0, ns, [x.ptr for x in W], [x.ptr for x in G], [x.ptr for x in M], [x.ptr for x in V],
                              0.9, 0.999, lr, p, seeds[:2])
    for i, n in enumerate(ns):
        dropped = hash_rng.lr_dropout_mask(n, seeds[i], p)
        got = W[i].get()
        assert np.array_equal(got[dropped], w0[i][dropped]) and np.all(got[~dropped] != w0[i][~dropped])
        assert 0.3 < dropped.mean() < 0.5
    # lr_dropout == 0 is the plain update and needs no seeds
    W, G, A = [DevArr(hip, x) for x in w0], [DevArr(hip, x) for x in g], [DevArr(hip, x) for x in a0]
    W2, G2, A2 = [DevArr(hip, x) for x in w0], [DevArr(hip, x) for x in g], [DevArr(hip, x) for x in a0]
    hip.sgd_update_multi_lrd(0, ns, [x.ptr for x in W], [x.ptr for x in G], [x.ptr for x in A], mom, lr, 1, 0.0, seeds)
    hip.sgd_update_multi(0, ns, [x.ptr for x in W2], [x.ptr for x in G2], [x.ptr for x in A2], mom, lr, 1)
    for i in range(2):
        assert np.array_equal(W[i].get(), W2[i].get())
    with pytest.raises(hip.HipException):
        hip.sgd_update_multi_lrd(0, ns, [x.ptr for x in W], [x.ptr for x in G], [x.ptr for x in A], mom, lr, 1, 1.5, seeds)
