import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch


def transpose(input_t, axes_order):
    """Permute axes (transpose.py:9-18)."""
    return transpose_op(input_t, axes_order)


def transpose_op(input_t, axes_order, output_t=None, is_add_to_output=False):
    """output_t / is_add_to_output as for matmul_op (transpose.py:60-83)."""
    is_add_to_output = False if output_t is None else is_add_to_output
    op = nc.Cacheton.get(_TransposeOp, input_t.shape, nc.TensorAxes(axes_order, input_t.shape.rank))
    fresh = output_t is None
    if fresh:
        output_t = nn.Tensor(op.info.output_shape)
        output_t._set_op_name('transpose')
        output_t._assign_gradfn(input_t, lambda O_t, dO_t: transpose_dI_gradfn(op, input_t, O_t, dO_t))
    elif output_t.shape.size != op.info.output_shape.size:
        raise ValueError(f'output_t must have size {op.info.output_shape.size}')
    beta = 1 if is_add_to_output else 0
    out_arg = output_t if is_add_to_output else (output_t, 'w')
    launch(lambda dev, i, o: api.transpose(dev, op.shape, op.axes, i, o, beta), (input_t, 'r'), out_arg)
    return output_t


def transpose_dI_gradfn(op, input_t, O_t, dO_t):
    # backward of a permutation is the inverse permutation, accumulated (transpose.py:85-87)
    transpose_op(dO_t, op.axes_order.inversed(), output_t=input_t.get_grad(), is_add_to_output=True)


def depth_to_space(input_t, size):
    """(N, C, H, W) -> (N, C/size^2, H*size, W*size)   (transpose.py:20-38)."""
    N, C, H, W = input_t.shape
    if size < 2:
        raise ValueError('size should be >= 2')
    if C % (size * size) != 0:
        raise ValueError(f'Unable to divide {C} channels by {size*size} !')
    OC = C // (size * size)
    return (input_t.reshape((N, size, size, OC, H, W)).transpose((0, 3, 4, 1, 5, 2))
            .reshape((N, OC, H * size, W * size)))


def space_to_depth(input_t, size):
    """(N, C, H, W) -> (N, C*size^2, H/size, W/size)   (transpose.py:40-58)."""
    N, C, H, W = input_t.shape
    if size < 2:
        raise ValueError('size should be >= 2')
    if H % size != 0:
        raise ValueError(f'Unable to divide {H} H by {size} !')
    if W % size != 0:
        raise ValueError(f'Unable to divide {W} W by {size} !')
    OH, OW = H // size, W // size
    return (input_t.reshape((N, C, OH, size, OW, size)).transpose((0, 3, 5, 1, 2, 4))
            .reshape((N, size * size * C, OH, OW)))


class _TransposeOp:
    def __init__(self, input_shape, axes_order):
        self.axes_order = axes_order
        self.info = nc.info.InfoTranspose(input_shape, axes_order)
        if input_shape.rank > 8:
            raise ValueError('transpose supports rank <= 8')
        self.shape = tuple(input_shape)
        self.axes = tuple(axes_order)
