import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch


def matmul_op(a_t, b_t, output_t=None, is_add_to_output=False):
    """Row-major matmul  A(...,M,K) x B(...,K,N) = (...,M,N)   (matmul.py:8-23).

     output_t           write into this tensor (any shape of equal size); no
                        gradient function is registered then
     is_add_to_output   accumulate into output_t instead of overwriting
    """
    return matmulc_op(b_t, a_t, output_t=output_t, is_add_to_output=is_add_to_output)


def matmul(a_t, b_t):
    """Row-major matmul  A(...,M,K) x B(...,K,N) = (...,M,N)   (matmul.py:24-30)."""
    return matmulc_op(b_t, a_t)


def matmul_bias_act(x_t, w_t, bias_t=None, leaky_relu_alpha=None):
    """leaky_relu(matmul(x, w) + bias, alpha) in one launch: x (..., rows, in_ch), w (..., in_ch, out_ch),
    bias (out_ch,) broadcast over the rows.

    A dense layer writes the first two steps as a product followed by a broadcast add (module/Dense.py:44-48,
    dual_wise_op.py:110-130), which costs an extra read + write pass over the output; here the product's epilogue adds
    bias[n] and applies the activation before its only store, which gives the same bits.  bias_t and
    leaky_relu_alpha are optional; alpha must be > 0 (the backward pass reads the sign of the pre-activation off the
    output).  Gradients: x and w as matmul (matmul.py:64-72), bias the sum of the pre-activation gradient over the
    rows, each accumulated."""
    from .conv2D import _EpilogueGrad
    op = nc.Cacheton.get(_MatmulOp, w_t.shape, x_t.shape, False)   # column-major naming: a = w (K, M), b = x (N, K)
    B, M, N, K = op.BATCH, op.M, op.N, op.K
    if bias_t is not None and tuple(bias_t.shape) != (M,):
        raise ValueError(f'bias shape {tuple(bias_t.shape)} does not match {M} output features')
    if leaky_relu_alpha is not None and not leaky_relu_alpha > 0:
        raise ValueError('leaky_relu_alpha must be > 0 for the fused form')
    act = api.ACT_NONE if leaky_relu_alpha is None else api.ACT_LEAKY_RELU
    alpha = 0.0 if leaky_relu_alpha is None else float(leaky_relu_alpha)
    output_t = nn.Tensor(op.output_shape)
    output_t._set_op_name('matmul_bias_act')
    epi = _EpilogueGrad(act, alpha, dims=lambda shape: (B * N, M, 1))
    if bias_t is not None:   # first, so that one pass forms the pre-activation gradient and sums it per feature
        output_t._assign_gradfn(bias_t, lambda O_t, dO_t: epi.bias(O_t, dO_t, bias_t))
    output_t._assign_gradfn(w_t, lambda O_t, dO_t: matmul_a_grad(w_t, x_t, epi.pre(O_t, dO_t)))
    output_t._assign_gradfn(x_t, lambda O_t, dO_t: matmul_b_grad(w_t, x_t, epi.pre(O_t, dO_t)))
    args = [(x_t, 'r'), (w_t, 'r')] + ([(bias_t, 'r')] if bias_t is not None else [])

    def run(dev, x, w, *rest):
        b, c = (rest[0], rest[1]) if bias_t is not None else (None, rest[0])
        api.gemm_bias_act(dev, 0, 0, B, N, M, K, x, K, N * K, w, M, K * M, b, act, alpha, c, M, N * M)
    launch(run, *args, (output_t, 'w'))
    return output_t


def matmulc_op(a_t, b_t, output_t=None, is_add_to_output=False):
    """Column-major naming of the same product (matmul.py:33-62):
    A(...,K,M) x B(...,N,K) = (...,N,M); in row-major storage this is
    C[N][M] = B[N][K] . A[K][M]."""
    is_add_to_output = False if output_t is None else is_add_to_output
    op = nc.Cacheton.get(_MatmulOp, a_t.shape, b_t.shape, is_add_to_output)
    skip_init = False
    if output_t is None:
        output_t = nn.Tensor(op.output_shape)
        output_t._set_op_name('matmul')
        output_t._assign_gradfn(a_t, lambda O_t, dO_t: matmul_a_grad(a_t, b_t, dO_t))
        output_t._assign_gradfn(b_t, lambda O_t, dO_t: matmul_b_grad(a_t, b_t, dO_t))
        skip_init = True
    elif output_t.shape.size != op.output_shape.size:
        raise ValueError(f'output_t must have size {op.output_shape.size}')
    B, M, N, K = op.BATCH, op.M, op.N, op.K
    beta = 1 if is_add_to_output else 0
    out_arg = (output_t, 'w') if (skip_init or not is_add_to_output) else output_t
    launch(lambda dev, a, b, c: api.gemm(dev, 0, 0, B, N, M, K, b, K, N * K, a, M, K * M, c, M, N * M, beta),
           (a_t, 'r'), (b_t, 'r'), out_arg)
    return output_t


def matmul_a_grad(a_t, b_t, dO_t):
    """a.grad[K][M] += b[N][K]^T . dO[N][M]   (matmul.py:64-67); the transposed
    operand is read in place, not materialised."""
    op = nc.Cacheton.get(_MatmulOp, a_t.shape, b_t.shape, False)
    B, M, N, K = op.BATCH, op.M, op.N, op.K
    grad_t, beta = nc.op.accumulate_target(a_t.get_grad())
    launch(lambda dev, b, do, da: api.gemm(dev, 1, 0, B, K, M, N, b, K, N * K, do, M, N * M, da, M, K * M, beta),
           (b_t, 'r'), (dO_t, 'r'), grad_t)


def matmul_b_grad(a_t, b_t, dO_t):
    """b.grad[N][K] += dO[N][M] . a[K][M]^T   (matmul.py:69-72)."""
    op = nc.Cacheton.get(_MatmulOp, a_t.shape, b_t.shape, False)
    B, M, N, K = op.BATCH, op.M, op.N, op.K
    grad_t, beta = nc.op.accumulate_target(b_t.get_grad())
    launch(lambda dev, do, a, db: api.gemm(dev, 0, 1, B, N, K, M, do, M, N * M, a, M, K * M, db, K, N * K, beta),
           (dO_t, 'r'), (a_t, 'r'), grad_t)


class _MatmulOp:
    """Shape plan (matmul.py:76-104), column-major naming: a is (...,K,M),
    b is (...,N,K)."""

    def __init__(self, a_shape, b_shape, is_add_to_output):
        if a_shape.rank != b_shape.rank:
            raise ValueError(f'Ranks are not equal. {a_shape.rank} != {b_shape.rank}')
        rank = a_shape.rank
        if rank < 2:
            raise ValueError('Tensors rank must be at least 2.')
        K, M = a_shape[-2], a_shape[-1]
        N, b_cols = b_shape[-2], b_shape[-1]
        if K != b_cols:
            raise ValueError('A_ROWS != B_COLS')
        batch = a_shape[0:-2].size if rank > 2 else 1
        b_batch = b_shape[0:-2].size if rank > 2 else 1
        if batch != b_batch:
            raise ValueError(f'BATCH size {batch} != {b_batch} in shapes {a_shape} {b_shape}')
        self.output_shape = nc.TensorShape((N, M)) if rank == 2 else nc.TensorShape(a_shape[:-2] + (N, M))
        self.M, self.N, self.K, self.BATCH = M, N, K, batch
