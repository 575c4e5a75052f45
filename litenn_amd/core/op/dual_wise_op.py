import litenn_amd as nn
import litenn_amd.core as nc
from ..hip import api, launch

_OPS = {'add': api.BIN_ADD, 'sub': api.BIN_SUB, 'mul': api.BIN_MUL}


def dual_wise_op(kind, a_t, b_t, output_t=None, is_add_to_output=False):
    """out (+)= a (op) b with numpy broadcasting (dual_wise_op.py:77-108).
    Gradients of a broadcast operand are summed over the broadcast axes
    (dual_wise_op.py:110-130)."""
    is_add_to_output = False if output_t is None else is_add_to_output
    info = nc.Cacheton.get(nc.info.InfoBroadcast, a_t.shape, b_t.shape)
    code = _OPS[kind]
    if info.output_shape.rank > 8:
        raise ValueError('broadcast ops support rank <= 8')
    if output_t is None:
        output_t = nn.Tensor(info.output_shape)
        output_t._set_op_name(kind)
        output_t._assign_gradfn(a_t, lambda O_t, dO_t: _operand_gradfn(kind, info, 0, a_t, b_t, dO_t))
        output_t._assign_gradfn(b_t, lambda O_t, dO_t: _operand_gradfn(kind, info, 1, a_t, b_t, dO_t))
    elif output_t.shape.size != info.output_shape.size:
        raise ValueError(f'output_t must have size {info.output_shape.size}')
    beta = 1 if is_add_to_output else 0
    src_out = output_t._get_top_reference_source()
    aliased = src_out is a_t._get_top_reference_source() or src_out is b_t._get_top_reference_source()
    out_arg = output_t if (is_add_to_output or aliased) else (output_t, 'w')
    o_s, a_s, b_s = tuple(info.output_shape), tuple(info.a_br_shape), tuple(info.b_br_shape)
    launch(lambda dev, a, b, o: api.binary_bcast(dev, code, o_s, a_s, b_s, a, b, o, beta), (a_t, 'r'), (b_t, 'r'), out_arg)
    return output_t


def _operand_gradfn(kind, info, which, a_t, b_t, dO_t):
    target = (a_t, b_t)[which]
    other = (b_t, a_t)[which]
    red = (info.a_shape_reduction_axes, info.b_shape_reduction_axes)[which]
    o_s = tuple(info.output_shape)
    if kind == 'mul':
        # d(target) = dO * other, still in the broadcast shape
        other_s = tuple((info.b_br_shape, info.a_br_shape)[which])
        if red.rank == 0:
            launch(lambda dev, do, ot, g: api.binary_bcast(dev, api.BIN_MUL, o_s, o_s, other_s, do, ot, g, 1),
                   (dO_t, 'r'), (other, 'r'), target.get_grad())
            return
        tmp = nn.Tensor(info.output_shape)
        launch(lambda dev, do, ot, g: api.binary_bcast(dev, api.BIN_MUL, o_s, o_s, other_s, do, ot, g, 0),
               (dO_t, 'r'), (other, 'r'), (tmp, 'w'))
        src, scale = tmp, 1.0
    else:
        src, scale = dO_t, (-1.0 if (kind == 'sub' and which == 1) else 1.0)
    if red.rank == 0:
        n = info.output_shape.size
        launch(lambda dev, s, g: api.ew_fwd(dev, api.EW_MUL_CONST, n, s, g, scale, 1), (src, 'r'), target.get_grad())
    else:
        # sum over the broadcast axes into the operand's gradient
        launch(lambda dev, s, g: api.reduce_sum(dev, o_s, tuple(red), scale, s, g, 1), (src, 'r'), target.get_grad())


def add_op(a_t, b_t, output_t=None, is_add_to_output=False): return dual_wise_op('add', a_t, b_t, output_t, is_add_to_output)
def add(a_t, b_t): return add_op(a_t, b_t)
def sub_op(a_t, b_t, output_t=None, is_add_to_output=False): return dual_wise_op('sub', a_t, b_t, output_t, is_add_to_output)
def sub(a_t, b_t): return sub_op(a_t, b_t)
def mul_op(a_t, b_t, output_t=None, is_add_to_output=False): return dual_wise_op('mul', a_t, b_t, output_t, is_add_to_output)
def mul(a_t, b_t): return mul_op(a_t, b_t)
