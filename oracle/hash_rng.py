"""CPU restatement of the reference's on-device random initialisers.  TEST INFRASTRUCTURE ONLY.

The reference fills a parameter tensor with a counter hash: element i is a function of (uint32)(i + seed) alone
(initializer/RandomUniform.py:13-27, RandomNormal.py:10-30), the hashes being the two PCG variants of its device
helper text (CLKernelHelper.py:210-228).  All integer work is modulo 2**32 and reproduced bit for bit.  The float
stages are single precision throughout: the reference builds every kernel with -cl-single-precision-constant
(minicl/CLDevice.py:93), so the mean / stddev / low / high it formats into the kernel text are float literals, and
`u*(high-low)+low` (RandomUniform.py:20) and `mean+n*stddev` (RandomNormal.py:24) are float expressions.  The
multiply-add is taken as contracted into one fused operation (OpenCL C allows it by default, and which one a vendor
compiler emits cannot be read off the reference: at most one float ulp rides on that choice).

Pinning.  The reference holds no output vector of these kernels and its OpenCL text cannot run here, so the
integer stream is PARITY UNPINNED against the reference's device output.  What tests/test_oracle_hash_rng.py does
fix, independently of the formulas below: hash_u32 is a permutation of the 32-bit integers (inverted step by step
with modular inverses computed by pow(), and collision-free on 2**22 consecutive counters, where a random function
would collide about 2000 times); hash_u32x2 is a permutation of pairs (same inversion); single-bit avalanche near
16 of 32 bits; uniform moments and a Kolmogorov-Smirnov test of both distributions against scipy.stats.
"""
import numpy as np

M32 = np.uint64(0xFFFFFFFF)


def _u32(x):
    return np.asarray(x, dtype=np.uint64) & M32


def hash_u32(v):
    """hash_uint_uint (CLKernelHelper.py:210-215): one LCG step, then PCG's RXS-M-XS output permutation."""
    v = _u32(v)
    state = _u32(v * np.uint64(747796405) + np.uint64(2891336453))
    word = _u32(((state >> ((state >> np.uint64(28)) + np.uint64(4))) ^ state) * np.uint64(277803737))
    return ((word >> np.uint64(22)) ^ word).astype(np.uint32)


def hash_u32x2(x, y):
    """hash_uint2_uint2 (CLKernelHelper.py:217-228)."""
    k, c, s = np.uint64(1664525), np.uint64(1013904223), np.uint64(16)
    x = _u32(_u32(x) * k + c)
    y = _u32(_u32(y) * k + c)
    x = _u32(x + y * k)
    y = _u32(y + x * k)
    x = x ^ (x >> s)
    y = y ^ (y >> s)
    x = _u32(x + y * k)
    y = _u32(y + x * k)
    x = x ^ (x >> s)
    y = y ^ (y >> s)
    return x.astype(np.uint32), y.astype(np.uint32)


def _unit(h):
    """(float)h * UIF with UIF = 1.0 / (float)0xffffffffU = 2**-32 (CLKernelHelper.py:209, 243-246)."""
    return h.astype(np.float32) * np.float32(2.0 ** -32)


def _counter(n, seed):
    return (np.arange(n, dtype=np.uint64) + np.uint64(seed)) & M32


def fma32(a, b, c):
    """round_to_float32(a*b + c) with a single rounding, for float32 arrays / scalars.  The product of two
    floats is exact in double; the double sum is corrected to round-to-odd with the exact error of the addition
    (two-sum), after which the narrowing to float32 rounds as if it had seen the exact value."""
    a, b, c = (np.asarray(v, np.float32).astype(np.float64) for v in (a, b, c))
    p = a * b
    s = p + c
    bb = s - p
    e = (p - (s - bb)) + (c - bb)
    bits = np.atleast_1d(s).copy().view(np.int64)
    inexact = (np.atleast_1d(e) != 0) & ((bits & 1) == 0) & np.isfinite(np.atleast_1d(s))
    away = np.signbit(np.atleast_1d(e)) == np.signbit(np.atleast_1d(s))   # the exact value lies farther from zero than s
    bits += np.where(inexact, np.where(away, 1, -1), 0)
    return bits.view(np.float64).reshape(np.shape(s)).astype(np.float32)


def random_uniform(n, seed, low=0.0, high=1.0):
    """O[gid] = hash_float_uint(gid+seed)*(high-low)+low in single precision (RandomUniform.py:17-21,
    CLDevice.py:93): span = (float)high - (float)low, then one fused multiply-add."""
    u = _unit(hash_u32(_counter(n, seed)))
    span = np.float32(high) - np.float32(low)
    return fma32(u, span, np.float32(low))


def lr_dropout_mask(n, seed, lr_dropout):
    """True where an optimizer kernel sets lr = 0 for element gid: hash_float_uint(gid+seed) <= lr_dropout in single
    precision (optimizer/Optimizer.py:199-202; the threshold is a float literal there, CLDevice.py:93)."""
    return _unit(hash_u32(_counter(n, seed))) <= np.float32(lr_dropout)


def random_normal(n, seed, mean=0.0, stddev=1.0):
    """Box-Muller on hash_float2_uint(gid+seed) (RandomNormal.py:14-24).  A zero first half gives inf, as there."""
    x, y = hash_u32x2(_counter(n, seed), np.ones(n, dtype=np.uint64))
    fx, fy = _unit(x), _unit(y)
    with np.errstate(divide='ignore'):
        r = np.sqrt(np.float32(-2.0) * np.log(fx, dtype=np.float32), dtype=np.float32)
    normal = r * np.cos(np.float32(2.0 * np.float32(3.14159274101257)) * fy, dtype=np.float32)
    return fma32(normal, np.float32(stddev), np.float32(mean))
