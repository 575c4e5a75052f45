"""litenn_amd: LiteNN's conv2D / matmul path on AMD MI355X (gfx950).

    import litenn_amd as nn

exposes the same names as `import litenn as nn` for the part of LiteNN that
this package provides: Tensor, nn.conv2D / nn.matmul and their autograd, the
Conv2D / Dense modules, the pointwise / reduction ops and SGD a convolutional
training step needs, nn.devices and nn.cleanup().  Device work goes through
liblitenn_hip.so (hand-written HIP kernels, C ABI in include/litenn_hip.h);
there is no CPU or OpenCL fallback.
"""
import litenn_amd.core

from litenn_amd.core.Tensor import (Tensor,
                                    Tensor_like,
                                    Tensor_zeros_like,
                                    Tensor_ones_like,
                                    Tensor_from_value,
                                    Tensor_sliced_from_value)

import litenn_amd.core.info
import litenn_amd.core.op

import litenn_amd.core.initializer as initializer

from litenn_amd.core.backward import backward

from litenn_amd.core.op.conv2D import conv2D
from litenn_amd.core.op.conv2DTranspose import conv2DTranspose
from litenn_amd.core.op.depthwise_conv2D import depthwise_conv2D
from litenn_amd.core.op.dual_wise_op import add, sub, mul
from litenn_amd.core.op.element_wise_op import (add_const, sub_const, mul_const, div_const,
                                                leaky_relu, relu, square)
from litenn_amd.core.op.matmul import matmul
from litenn_amd.core.op.reduce import reduce_mean, reduce_sum
from litenn_amd.core.op.reshape import flatten, reshape
from litenn_amd.core.op.transpose import depth_to_space, space_to_depth, transpose
from litenn_amd.core.op.unfold2D import unfold2D

from litenn_amd.core import devices

from litenn_amd.core.module.Module import Module
from litenn_amd.core.module.Conv2D import Conv2D
from litenn_amd.core.module.Conv2DTranspose import Conv2DTranspose
from litenn_amd.core.module.DepthwiseConv2D import DepthwiseConv2D
from litenn_amd.core.module.SeparableConv2D import SeparableConv2D
from litenn_amd.core.module.Dense import Dense

import litenn_amd.core.optimizer as optimizer


def cleanup():
    """Drop cached plans and hints and release all device memory of the
    current devices.  No Tensor may be alive (litenn/__init__.py:117-125)."""
    litenn_amd.core.Cacheton._cleanup()
    if Tensor._object_count != 0:
        raise Exception(f'Unable to cleanup while {Tensor._object_count} Tensor objects exist.')
    devices.cleanup()
