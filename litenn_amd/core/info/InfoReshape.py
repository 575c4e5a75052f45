from ..TensorShape import TensorShape


class InfoReshape:
    """.output_shape for reshaping `shape` to `target_shape`, which may hold
    one -1 (InfoReshape.py:23-44; integer arithmetic throughout)."""
    __slots__ = ['output_shape']

    def __init__(self, shape, target_shape):
        out, remain, unknown = [], shape.size, None
        for t in target_shape:
            t = int(t)
            if t == -1:
                if unknown is not None:
                    raise ValueError('Can specify only one unknown dimension.')
                unknown = len(out)
            else:
                if t < 1 or remain % t != 0:
                    raise ValueError(f'Cannot reshape {shape} to {target_shape}.')
                remain //= t
            out.append(t)
        if unknown is not None:
            out[unknown] = remain
        elif remain != 1:
            raise ValueError(f'Cannot reshape {shape} to {target_shape}.')
        self.output_shape = TensorShape(out)
