from collections.abc import Iterable


class TensorAxes(Iterable):
    """Validated, immutable tuple of distinct axis indices, or the special
    "all axes" value built from None (same contract as TensorAxes.py:3-157).

     axes         TensorAxes | int | iterable of ints | None
     shape_rank   needed when axes may hold negative values

    A + B concatenates, A - B removes B's axes from A.
    """
    __slots__ = ['axes', 'rank', '_inversed']

    def __init__(self, axes, shape_rank=None):
        self._inversed = None
        if isinstance(axes, TensorAxes):
            self.axes, self.rank, self._inversed = axes.axes, axes.rank, axes._inversed
            return
        if axes is None:
            self.axes = self.rank = None
            return
        if not isinstance(axes, Iterable):
            axes = (axes,)
        seen = []
        for x in axes:
            if x is None:
                raise ValueError(f'Incorrent value {x} in axes {axes}')
            x = int(x)
            if x < 0:
                if shape_rank is None:
                    raise ValueError(f'Incorrent value {x} in axes {axes}, or provide shape_rank')
                x += shape_rank
            if x in seen:
                raise ValueError('Axes must contain unique values.')
            seen.append(x)
        self.axes = tuple(seen)
        self.rank = len(seen)

    def is_none_axes(self):
        return self.axes is None

    def _require(self, what):
        if self.axes is None:
            raise Exception(f'none-axes does not support {what}. Handle none-axes by calling .is_none_axes()')

    def sorted(self):
        return TensorAxes(sorted(self.axes))

    def inversed(self):
        """Axes order that undoes this one: (0,2,3,1) -> (0,3,1,2)."""
        self._require('inversed()')
        if self._inversed is None:
            if sorted(self.axes) != list(range(self.rank)):
                raise Exception(f'axes {self.axes} are inconsistent to do inverse order.')
            inv = [0] * self.rank
            for pos, axis in enumerate(self.axes):
                inv[axis] = pos
            self._inversed = TensorAxes(inv)
        return self._inversed

    def __hash__(self): return hash(self.axes)

    def __eq__(self, other):
        if isinstance(other, TensorAxes):
            return self.axes == other.axes
        if isinstance(other, Iterable):
            return self.axes == tuple(other)
        return False

    def __iter__(self):
        self._require('iteration')
        return iter(self.axes)

    def __len__(self): return self.rank

    def __getitem__(self, key):
        self._require('indexing')
        if isinstance(key, slice):
            return TensorAxes(self.axes[key])
        return self.axes[key]

    def __add__(self, o):
        if not isinstance(o, Iterable):
            raise ValueError(f'unable to use type {o.__class__} in TensorAxes append')
        return TensorAxes(self.axes + tuple(o))

    def __radd__(self, o):
        if not isinstance(o, Iterable):
            raise ValueError(f'unable to use type {o.__class__} in TensorAxes append')
        return TensorAxes(tuple(o) + self.axes)

    def __sub__(self, o):
        if not isinstance(o, Iterable):
            raise ValueError(f'unable to use type {o.__class__} in TensorAxes substraction')
        drop = tuple(o)
        return TensorAxes([a for a in self.axes if a not in drop])

    def __rsub__(self, o):
        if not isinstance(o, Iterable):
            raise ValueError(f'unable to use type {o.__class__} in TensorAxes substraction')
        return TensorAxes([a for a in o if a not in self.axes])

    def __str__(self): return '(None)' if self.axes is None else str(self.axes)
    def __repr__(self): return 'TensorAxes' + str(self)
