class InfoTranspose:
    """.output_shape = shape permuted by axes_order; .no_changes when the
    order is the identity (InfoTranspose.py:27-33)."""
    __slots__ = ['no_changes', 'output_shape']

    def __init__(self, shape, axes_order):
        if shape.rank != axes_order.rank:
            raise ValueError('axes must match the shape')
        self.output_shape = shape[axes_order]
        self.no_changes = axes_order == shape.axes_arange()
