"""Pins the matmul oracle (matmul.py:8-72, test matmul.py:167-234)."""
import numpy as np
import pytest

from oracle import matmul_fwd, matmul_da, matmul_db


def _case(rs):
    # same generator as the reference's self-test, with the K*N cap lowered
    batch = rs.randint(8) + 1
    M = rs.randint(8) + 1
    N = rs.randint(32768) + 1
    K = rs.randint(32768) + 1
    while K * N > 200000 // batch:
        K, N = max(1, K // 2), max(1, N // 2)
    if rs.randint(2) == 0:
        size = [2, 4, 8, 16][rs.randint(4)]
        M, N, K = (max(1, v // size) * size for v in (M, N, K))
    return batch, M, N, K


def test_integer_exact_and_shapes():
    rs = np.random.RandomState(0)
    for _ in range(20):
        batch, M, N, K = _case(rs)
        ash, bsh = ((M, K), (K, N)) if batch == 1 else ((batch, M, K), (batch, K, N))
        a = rs.randint(16, size=ash).astype(np.float32)
        b = rs.randint(16, size=bsh).astype(np.float32)
        c = matmul_fwd(a, b)
        ref = np.matmul(a.astype(np.float64), b.astype(np.float64))
        assert c.shape == ref.shape and np.array_equal(c, ref)
        dc = rs.randint(8, size=c.shape).astype(np.float32)
        da, db = matmul_da(dc, b, a.shape), matmul_db(a, dc, b.shape)
        assert np.array_equal(da, np.matmul(dc.astype(np.float64), np.swapaxes(b, -1, -2)))
        assert np.array_equal(db, np.matmul(np.swapaxes(a, -1, -2).astype(np.float64), dc))
        # adjoints, exact in integers
        assert (c * dc).sum() == (a * da).sum() == (b * db).sum()


def test_shape_errors():
    with pytest.raises(ValueError):
        matmul_fwd(np.zeros((2, 3)), np.zeros((1, 3, 4)))
    with pytest.raises(ValueError):
        matmul_fwd(np.zeros((3,)), np.zeros((3,)))
    with pytest.raises(ValueError):
        matmul_fwd(np.zeros((2, 3)), np.zeros((4, 5)))
    with pytest.raises(ValueError):
        matmul_fwd(np.zeros((2, 2, 3)), np.zeros((3, 3, 4)))
