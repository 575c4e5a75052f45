from ..TensorShape import TensorShape


class InfoReduction:
    """Shapes of a reduction over `axes` (InfoReduction.py:25-50).

    .reduction_axes (sorted)  .output_axes (the rest)
    .output_shape   .output_shape_keepdims
    """
    __slots__ = ['reduction_axes', 'output_axes', 'output_shape', 'output_shape_keepdims']

    def __init__(self, shape, axes, keepdims):
        all_axes = shape.axes_arange()
        if axes.is_none_axes():
            axes = all_axes
        for axis in axes:
            if axis not in all_axes:
                raise ValueError(f'Wrong axis {axis} not in {all_axes}')
        self.reduction_axes = axes.sorted()
        self.output_axes = all_axes - axes
        self.output_shape_keepdims = TensorShape(1 if a in self.reduction_axes else shape[a]
                                                 for a in range(shape.rank))
        if keepdims:
            self.output_shape = self.output_shape_keepdims
        elif self.output_axes.rank == 0:
            self.output_shape = TensorShape((1,))
        else:
            self.output_shape = shape[self.output_axes]
