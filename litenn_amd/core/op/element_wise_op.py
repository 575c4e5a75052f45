import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch

# The reference builds pointwise kernels from C snippets at run time
# (element_wise_op.py:48-110).  Here the ops a conv-net training step needs
# around the contraction kernels are prebuilt; user-supplied kernel text is
# not supported.
_OPS = {
    'add_const': api.EW_ADD_CONST,
    'mul_const': api.EW_MUL_CONST,
    'leaky_relu': api.EW_LEAKY_RELU,
    'square': api.EW_SQUARE,
    'relu': api.EW_RELU,
}


def element_wise_op(kind, param, input_t, output_t=None, is_add_to_output=False):
    """out (+)= f(in); when no output_t is given a new tensor is made and
    its gradient function does in.grad += f'(in) * dout (element_wise_op.py:48-81)."""
    is_add_to_output = False if output_t is None else is_add_to_output
    code = _OPS[kind]
    n = input_t.shape.size
    if output_t is None:
        output_t = nn.Tensor(input_t.shape)
        output_t._set_op_name(kind if kind in ('square', 'relu') else f'{kind}({param})' if kind == 'leaky_relu' else kind)
        output_t._assign_gradfn(input_t, lambda O_t, dO_t: _input_gradfn(code, param, input_t, dO_t))
    elif output_t.shape.size != n:
        raise ValueError(f'output_t must have size {n}')
    beta = 1 if is_add_to_output else 0
    in_place = output_t._get_top_reference_source() is input_t._get_top_reference_source()
    out_arg = output_t if (is_add_to_output or in_place) else (output_t, 'w')
    launch(lambda dev, i, o: api.ew_fwd(dev, code, n, i, o, param, beta), (input_t, 'r'), out_arg)
    return output_t


def _input_gradfn(code, param, input_t, dO_t):
    n = input_t.shape.size
    grad_t, beta = nc.op.accumulate_target(input_t.get_grad())
    launch(lambda dev, i, do, di: api.ew_bwd(dev, code, n, i, do, di, param, beta), (input_t, 'r'), (dO_t, 'r'), grad_t)


def add_const_op(input_t, value, output_t=None, is_add_to_output=False):
    return element_wise_op('add_const', float(value), input_t, output_t, is_add_to_output)
def add_const(input_t, value): return add_const_op(input_t, value)
def sub_const_op(input_t, value, output_t=None, is_add_to_output=False):
    return add_const_op(input_t, -value, output_t, is_add_to_output)
def sub_const(input_t, value): return add_const(input_t, -value)
def mul_const_op(input_t, value, output_t=None, is_add_to_output=False):
    return element_wise_op('mul_const', float(value), input_t, output_t, is_add_to_output)
def mul_const(input_t, value): return mul_const_op(input_t, value)
def div_const_op(input_t, value, output_t=None, is_add_to_output=False):
    return mul_const_op(input_t, 1.0 / value, output_t, is_add_to_output)
def div_const(input_t, value): return mul_const(input_t, 1.0 / value)
def leaky_relu_op(input_t, alpha, output_t=None, is_add_to_output=False):
    return element_wise_op('leaky_relu', float(alpha), input_t, output_t, is_add_to_output)
def leaky_relu(input_t, alpha=0.1):
    """x >= 0 ? x : alpha*x   (element_wise_op.py:208-222)."""
    return leaky_relu_op(input_t, alpha)
def relu_op(input_t, output_t=None, is_add_to_output=False):
    return element_wise_op('relu', 0.0, input_t, output_t, is_add_to_output)
def relu(input_t): return relu_op(input_t)
def square_op(input_t, output_t=None, is_add_to_output=False):
    return element_wise_op('square', 0.0, input_t, output_t, is_add_to_output)
def square(input_t):
    """x*x   (element_wise_op.py:331-344)."""
    return square_op(input_t)
