from ..TensorAxes import TensorAxes
from ..TensorShape import TensorShape


class InfoBroadcast:
    """numpy-style broadcast of two shapes (InfoBroadcast.py:40-86).

    .a_br_shape / .b_br_shape   operands left-padded with ones to equal rank
    .output_shape               broadcast result
    .a_shape_reduction_axes     axes to sum over to get a's gradient back
    .b_shape_reduction_axes     likewise for b
    .a_tiles / .b_tiles         repeat counts per axis
    """
    __slots__ = ['a_br_shape', 'a_shape_reduction_axes', 'a_tiles', 'b_br_shape', 'b_shape_reduction_axes',
                 'b_tiles', 'output_shape']

    def __init__(self, a_shape, b_shape):
        rank = max(a_shape.rank, b_shape.rank)
        a_br = (1,) * (rank - a_shape.rank) + a_shape
        b_br = (1,) * (rank - b_shape.rank) + b_shape
        out, a_red, b_red = [], [], []
        a_tiles, b_tiles = [1] * rank, [1] * rank
        for axis, (x, y) in enumerate(zip(a_br, b_br)):
            if x != y:
                if x == 1:
                    a_tiles[axis] = y
                    a_red.append(axis)
                elif y == 1:
                    b_tiles[axis] = x
                    b_red.append(axis)
                else:
                    raise ValueError(f'operands could not be broadcast together with shapes {a_shape} {b_shape}')
            out.append(max(x, y))
        self.output_shape = TensorShape(out)
        self.a_br_shape, self.b_br_shape = a_br, b_br
        self.a_shape_reduction_axes, self.b_shape_reduction_axes = TensorAxes(a_red), TensorAxes(b_red)
        self.a_tiles, self.b_tiles = tuple(a_tiles), tuple(b_tiles)
