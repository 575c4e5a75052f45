"""Optimizers (nn.optimizer.*): SGD and Adam."""
import litenn_amd as nn

from .Optimizer import Optimizer
from .SGD import SGD
from .Adam import Adam


class freeze:
    """`with nn.optimizer.freeze():` - optimizer-attached tensors used by ops
    created inside the block receive no gradient (optimizer/__init__.py:9-23)."""

    def __enter__(self):
        nn.Tensor._freeze_stack += 1

    def __exit__(self, *exc):
        nn.Tensor._freeze_stack -= 1
        if nn.Tensor._freeze_stack < 0:
            raise ValueError('Wrong _freeze_stack')
