from collections.abc import Iterable

from .TensorAxes import TensorAxes


class TensorShape(Iterable):
    """Validated, immutable tensor shape: every extent is an int >= 1 and the
    empty shape becomes (1,) (same contract as TensorShape.py:4-101).

    attributes: .shape (tuple) .size (product) .rank
    """
    __slots__ = ['shape', 'size', 'rank']

    def __init__(self, shape):
        if isinstance(shape, TensorShape):
            self.shape, self.size, self.rank = shape.shape, shape.size, shape.rank
            return
        if isinstance(shape, (int, float)):
            shape = (int(shape),)
        if not isinstance(shape, Iterable):
            raise ValueError('Invalid type to create TensorShape')
        dims, size = [], 1
        for x in shape:
            if x is None or int(x) < 1:
                raise ValueError(f'Incorrent value {x} in shape {shape}')
            dims.append(int(x))
            size *= int(x)
        if not dims:
            dims = [1]
        self.shape = tuple(dims)
        self.rank = len(dims)
        self.size = size

    def axes_arange(self):
        """TensorAxes (0, 1, ..., rank-1)."""
        return TensorAxes(range(self.rank))

    def transpose_by_axes(self, axes):
        return TensorShape(self.shape[a] for a in TensorAxes(axes))

    def __hash__(self): return hash(self.shape)

    def __eq__(self, other):
        if isinstance(other, TensorShape):
            return self.shape == other.shape
        if isinstance(other, Iterable):
            return self.shape == tuple(other)
        return False

    def __iter__(self): return iter(self.shape)
    def __len__(self): return self.rank

    def __getitem__(self, key):
        if isinstance(key, TensorAxes) and key.is_none_axes():
            return self
        if isinstance(key, Iterable):
            return self.transpose_by_axes(key)
        if isinstance(key, slice):
            return TensorShape(self.shape[key])
        return self.shape[key]

    def __add__(self, o):
        if not isinstance(o, Iterable):
            raise ValueError(f'unable to use type {o.__class__} in TensorShape append')
        return TensorShape(self.shape + tuple(o))

    def __radd__(self, o):
        if not isinstance(o, Iterable):
            raise ValueError(f'unable to use type {o.__class__} in TensorShape append')
        return TensorShape(tuple(o) + self.shape)

    def __str__(self): return str(self.shape)
    def __repr__(self): return 'TensorShape' + str(self)
