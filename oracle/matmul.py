"""matmul forward / dA / dB oracle (test infrastructure only).

Restates the user-level contract of litenn/core/op/matmul.py:8-72:
row-major C[..., M, N] = A[..., M, K] @ B[..., K, N] (matmul.py:24-30), with
dA += dC @ B^T (matmul.py:69-72 in the kernel's column-major naming) and
dB += A^T @ dC (matmul.py:64-67).  Shape rules of matmul.py:78-100.
"""
import numpy as np


def _check(a_shape, b_shape):
    if len(a_shape) != len(b_shape):
        raise ValueError(f'Ranks are not equal. {len(a_shape)} != {len(b_shape)}')
    if len(a_shape) < 2:
        raise ValueError('Tensors rank must be at least 2.')
    if a_shape[-1] != b_shape[-2]:
        raise ValueError('A_ROWS != B_COLS')
    if int(np.prod(a_shape[:-2], dtype=np.int64)) != int(np.prod(b_shape[:-2], dtype=np.int64)):
        raise ValueError('BATCH size mismatch')


def matmul_fwd(a, b, dtype=np.float64):
    _check(a.shape, b.shape)
    M, K = a.shape[-2:]
    N = b.shape[-1]
    a3 = a.astype(dtype).reshape(-1, M, K)
    b3 = b.astype(dtype).reshape(-1, K, N)
    # the reference's output keeps the leading dims of its first kernel
    # operand, which is the user's B (matmul.py:23,97-100)
    lead = b.shape[:-2]
    return np.matmul(a3, b3).reshape(lead + (M, N))


def matmul_da(dc, b, a_shape, dtype=np.float64):
    M, K = a_shape[-2:]
    N = b.shape[-1]
    d3 = dc.astype(dtype).reshape(-1, M, N)
    b3 = b.astype(dtype).reshape(-1, K, N)
    return np.matmul(d3, b3.transpose(0, 2, 1)).reshape(a_shape)


def matmul_db(a, dc, b_shape, dtype=np.float64):
    M, K = a.shape[-2:]
    N = b_shape[-1]
    a3 = a.astype(dtype).reshape(-1, M, K)
    d3 = dc.astype(dtype).reshape(-1, M, N)
    return np.matmul(a3.transpose(0, 2, 1), d3).reshape(b_shape)
