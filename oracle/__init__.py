"""CPU oracle for the conv2D / matmul hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module: it exists so that tests, the smoke check and the CPU-baseline leg of
the benchmark can compare the HIP path against an independent restatement of
the reference algorithm.  Each function cites the reference file:line
(relative to the litenn source tree) whose behaviour it restates.

Pinning status (what checks each function, independent of its own formula):

  info_conv2d        closed-form invariants, the textbook floor formula, and
                     the literal shape table of the benchmark configurations
                     (tests/test_oracle_info.py)
  unfold index maps  brute-force nested loops over the reference's own test
                     grid + exact integer adjoint identity
                     (tests/test_oracle_unfold.py)
  conv fwd/dX/dW     scipy.signal.correlate2d, explicit loop restatement of
                     the reference's numpy checker, adjoint identities,
                     1x1 == einsum, full-kernel 'valid' == matmul
                     (tests/test_oracle_conv.py)
  conv2DTranspose    scatter-form definition loops (exact on integers), the
   fwd/dI/dK         adjoint identity against the pinned conv2D oracle,
                     linearity in the kernel, stride-1 == conv2D with the
                     kernel flipped and its channel axes swapped
                     (tests/test_oracle_conv_transpose.py)
  depthwise          equals the pinned conv2D oracle applied to a kernel that is
   fwd/dI/dK         zero off the channel diagonal (forward, dI, and the
                     diagonal of dK), exact on integers
                     (tests/test_oracle_depthwise.py)
  matmul fwd/dA/dB   np.matmul fp64 on integer-valued data (exact) and
                     adjoint identities (tests/test_oracle_matmul.py)
  refpath (C, fp32)  must reproduce the fp64 oracle exactly on integer-valued
                     data and within 1e-5 on random data
                     (tests/test_oracle_refpath.py)

  hash_rng           integer hashes: permutation property by independent inversion,
                     no collisions over 2**22 counters, avalanche; float stages:
                     moments and Kolmogorov-Smirnov against scipy.stats
                     (tests/test_oracle_hash_rng.py).  PARITY UNPINNED against the
                     reference's device output: the reference holds no vector of
                     these kernels and its OpenCL text cannot run here.

No other function here is "parity unpinned".
"""
from .conv_info import info_conv2d, ConvInfo                      # noqa: F401
from .unfold import (unfold_index_map, unfold_T_index_map,        # noqa: F401
                     apply_index_map)
from .conv import conv2d_fwd, conv2d_dx, conv2d_dw, conv2d_all    # noqa: F401
from .conv_transpose import (conv2d_transpose_fwd, conv2d_transpose_di,   # noqa: F401
                             conv2d_transpose_dk, conv2d_transpose_all)
from .depthwise import depthwise_fwd, depthwise_di, depthwise_dk, depthwise_all   # noqa: F401
from .matmul import matmul_fwd, matmul_da, matmul_db              # noqa: F401
