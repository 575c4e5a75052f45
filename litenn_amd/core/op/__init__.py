from ..hip import HipDevicesBuffers


def accumulate_target(grad_t):
    """How to add into a gradient tensor: (launch argument, beta).  A gradient
    whose storage has not been touched yet is all zeros by definition
    (Tensor.get_grad), so the first contribution may overwrite it (beta 0,
    skipping the zero fill and the read-modify-write); later ones accumulate."""
    if all(not b.has_ptr() for b in grad_t._get_buffers()):
        return (grad_t, 'w'), 0
    return grad_t, 1


from .conv2D import conv2D, conv2D_bias_act
from .conv2DTranspose import conv2DTranspose
from .depthwise_conv2D import depthwise_conv2D
from .element_wise_op import (element_wise_op,
                              add_const_op as add_const,
                              div_const_op as div_const,
                              leaky_relu_op as leaky_relu,
                              mul_const_op as mul_const,
                              relu_op as relu,
                              square_op as square,
                              sub_const_op as sub_const)
from .dual_wise_op import (dual_wise_op,
                           add_op as add,
                           sub_op as sub,
                           mul_op as mul)
from .matmul import (matmul_op as matmul,
                     matmulc_op as matmulc,
                     matmul_bias_act)
from .reduce import (reduce_mean_op as reduce_mean,
                     reduce_sum_op as reduce_sum)
from .reshape import reshape
from .transpose import transpose_op as transpose
from .unfold2D import unfold2D
