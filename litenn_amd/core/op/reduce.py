import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch


def reduce_op(op_type, input_t, axes=None, keepdims=False, output_t=None, is_add_to_output=False):
    """'sum' or 'mean' over `axes` (None = all) (reduce.py:166-205).  One
    strided reduction kernel replaces the reference's transpose, log2 staged
    in-place halving and slice (reduce.py:192-203)."""
    if op_type not in ('sum', 'mean'):
        raise ValueError(f"reduce '{op_type}' is outside the conv2D / matmul path of this package")
    is_add_to_output = False if output_t is None else is_add_to_output
    op = nc.Cacheton.get(_ReduceOp, op_type, input_t.shape, nc.TensorAxes(axes, input_t.shape.rank), keepdims)
    if output_t is None:
        output_t = nn.Tensor(op.info.output_shape)
        output_t._op = op
        output_t._set_op_name(f'reduce_{op_type}')
        output_t._assign_gradfn(input_t, lambda O_t, dO_t: reduce_dI_gradfn(op, input_t, O_t, dO_t))
    elif output_t.shape.size != op.info.output_shape.size:
        raise ValueError(f'output_t must have size {op.info.output_shape.size}')
    beta = 1 if is_add_to_output else 0
    out_arg = output_t if is_add_to_output else (output_t, 'w')
    launch(lambda dev, i, o: api.reduce_sum(dev, op.shape, op.axes, op.scale, i, o, beta), (input_t, 'r'), out_arg)
    return output_t


def reduce_dI_gradfn(op, input_t, O_t, dO_t):
    # in.grad[idx] += dO[idx with reduced axes dropped] (/ count for mean)   (reduce.py:243-255)
    grad_t, beta = nc.op.accumulate_target(input_t.get_grad())
    launch(lambda dev, do, di: api.reduce_sum_bwd(dev, op.shape, op.axes, op.scale, do, di, beta), (dO_t, 'r'), grad_t)


class _ReduceOp:
    def __init__(self, op_type, input_shape, axes, keepdims=False):
        self.op_type = op_type
        self.info = info = nc.info.InfoReduction(input_shape, axes, keepdims)
        if input_shape.rank > 8:
            raise ValueError('reductions support rank <= 8')
        self.shape = tuple(input_shape)
        self.axes = tuple(info.reduction_axes)
        count = 1
        for a in self.axes:
            count *= input_shape[a]
        self.COLS = count
        self.scale = 1.0 / count if op_type == 'mean' else 1.0


def reduce_sum_op(input_t, axes=None, keepdims=False, output_t=None, is_add_to_output=False):
    return reduce_op('sum', input_t, axes, keepdims, output_t, is_add_to_output)
def reduce_sum(input_t, axes=None, keepdims=False): return reduce_sum_op(input_t, axes, keepdims)
def reduce_mean_op(input_t, axes=None, keepdims=False, output_t=None, is_add_to_output=False):
    return reduce_op('mean', input_t, axes, keepdims, output_t, is_add_to_output)
def reduce_mean(input_t, axes=None, keepdims=False): return reduce_mean_op(input_t, axes, keepdims)
