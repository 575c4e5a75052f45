"""ctypes binding of liblitenn_hip.so, the C ABI declared in include/litenn_hip.h.

Takes the place of the reference's OpenCL binding
(litenn/core/minicl/api/OpenCL/OpenCL.py:16-23 loads libOpenCL and
:175-198 maps status codes to exceptions).  Pure Python + numpy; the library
is built in-tree by `make -C litenn_amd/csrc` and there is no fallback: if it
is missing, importing this module raises.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get('LITENN_HIP_LIB',
                          os.path.normpath(os.path.join(_HERE, '..', '..', 'liblitenn_hip.so')))

OK, ERR_INVALID, ERR_OOM, ERR_NO_DEVICE, ERR_HIP, ERR_UNSUPPORTED = 0, -1, -2, -3, -4, -5
_NAMES = {ERR_INVALID: 'INVALID', ERR_OOM: 'OUT_OF_MEMORY', ERR_NO_DEVICE: 'NO_DEVICE',
          ERR_HIP: 'HIP_ERROR', ERR_UNSUPPORTED: 'UNSUPPORTED'}

EW_ADD_CONST, EW_MUL_CONST, EW_LEAKY_RELU, EW_SQUARE, EW_RELU = range(5)
BIN_ADD, BIN_SUB, BIN_MUL = range(3)


class HipException(Exception):
    """A failed library call.  .code is the negative status, .message the
    library's text (role of CL.Exception, OpenCL.py:186-198)."""

    def __init__(self, code, message):
        self.code = code
        self.message = message
        super().__init__(f'{_NAMES.get(code, code)}: {message}')


class ConvDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ('N', 'C', 'IH', 'IW', 'O', 'KH', 'KW', 'OH', 'OW', 'PADL', 'PADT', 'stride', 'dilation')]


_c_int, _c_u32, _c_u64, _c_i64, _c_f32 = ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int64, ctypes.c_float
_c_f64 = ctypes.c_double
_ptr = ctypes.c_void_p
_i32arr = ctypes.POINTER(ctypes.c_int32)

# name -> argument types (every function returns int except lnn_last_error)
SIGNATURES = {
    'lnn_device_count': [ctypes.POINTER(_c_int)],
    'lnn_device_info': [_c_int, ctypes.c_char_p, _c_int, ctypes.POINTER(_c_u64), ctypes.POINTER(_c_int),
                        ctypes.POINTER(_c_int)],
    'lnn_release_device': [_c_int],
    'lnn_malloc': [_c_int, _c_u64, ctypes.POINTER(_ptr)],
    'lnn_free': [_c_int, _ptr],
    'lnn_mem_info': [_c_int, ctypes.POINTER(_c_u64), ctypes.POINTER(_c_u64)],
    'lnn_memcpy_h2d': [_c_int, _ptr, _ptr, _c_u64],
    'lnn_memcpy_d2h': [_c_int, _ptr, _ptr, _c_u64],
    'lnn_memcpy_d2d': [_c_int, _ptr, _ptr, _c_u64],
    'lnn_fill_u32': [_c_int, _ptr, _c_u32, _c_u64],
    'lnn_synchronize': [_c_int],
    'lnn_event_create': [_c_int, ctypes.POINTER(_ptr)],
    'lnn_event_record': [_c_int, _ptr],
    'lnn_event_elapsed_ms': [_c_int, _ptr, _ptr, ctypes.POINTER(_c_f32)],
    'lnn_event_destroy': [_c_int, _ptr],
    'lnn_gemm_f32': [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _ptr, _c_int, _c_i64,
                     _ptr, _c_int, _c_i64, _ptr, _c_int, _c_i64, _c_int],
    'lnn_gemm_bias_act_f32': [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _ptr, _c_int, _c_i64,
                              _ptr, _c_int, _c_i64, _ptr, _c_int, _c_f32, _ptr, _c_int, _c_i64],
    'lnn_conv2d_fwd_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_fwd_bias_act_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int, ctypes.c_float, _ptr],
    'lnn_depthwise_conv2d_fwd_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_depthwise_conv2d_dgrad_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_depthwise_conv2d_wgrad_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_dgrad_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_wgrad_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_weights_plan': [ctypes.POINTER(ConvDesc), _c_int, ctypes.POINTER(_c_int)],
    'lnn_conv2d_permute_weights_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _c_int, _ptr],
    'lnn_conv2d_fwd_pw_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int, ctypes.c_float, _ptr, _c_int],
    'lnn_conv2d_dgrad_pw_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_wgrad_iohw_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_wgrad_noalloc_f32': [_c_int, ctypes.POINTER(ConvDesc), _ptr, _ptr, _ptr, _c_int],
    'lnn_conv2d_fwd_path': [ctypes.POINTER(ConvDesc), _c_int, ctypes.POINTER(_c_int)],
    'lnn_conv2d_wgrad_last_plan': [_c_int, _i32arr],
    'lnn_conv2d_dgrad_path': [ctypes.POINTER(ConvDesc), _c_int, _c_int, ctypes.POINTER(_c_int), _i32arr],
    'lnn_unfold2d_f32': [_c_int] + [_c_int] * 14 + [_ptr, _ptr, _c_int],
    'lnn_transpose_f32': [_c_int, _c_int, _i32arr, _i32arr, _ptr, _ptr, _c_int],
    'lnn_ew_fwd_f32': [_c_int, _c_int, _c_u64, _ptr, _ptr, _c_f32, _c_int],
    'lnn_ew_bwd_f32': [_c_int, _c_int, _c_u64, _ptr, _ptr, _ptr, _c_f32, _c_int],
    'lnn_binary_bcast_f32': [_c_int, _c_int, _c_int, _i32arr, _i32arr, _i32arr, _ptr, _ptr, _ptr, _c_int],
    'lnn_reduce_sum_f32': [_c_int, _c_int, _i32arr, _c_u32, _c_f32, _ptr, _ptr, _c_int],
    'lnn_reduce_sum_bwd_f32': [_c_int, _c_int, _i32arr, _c_u32, _c_f32, _ptr, _ptr, _c_int],
    'lnn_sgd_update_f32': [_c_int, _c_u64, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_int],
    'lnn_adam_update_f32': [_c_int, _c_u64, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_f32],
    'lnn_sgd_update_multi_f32': [_c_int, _c_int, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_int],
    'lnn_adam_update_multi_f32': [_c_int, _c_int, _ptr, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_f32],
    'lnn_sgd_update_multi_wp_f32': [_c_int, _c_int, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_int, _ptr, _ptr, _ptr, _ptr],
    'lnn_adam_update_multi_wp_f32': [_c_int, _c_int, _ptr, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_f32, _ptr, _ptr, _ptr, _ptr],
    'lnn_sgd_update_multi_lrd_f32': [_c_int, _c_int, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_int, _c_f32, _ptr, _ptr, _ptr, _ptr, _ptr],
    'lnn_adam_update_multi_lrd_f32': [_c_int, _c_int, _ptr, _ptr, _ptr, _ptr, _ptr, _c_f32, _c_f32, _c_f32, _c_f32, _ptr, _ptr, _ptr, _ptr, _ptr],
    'lnn_bias_act_bwd_f32': [_c_int, _c_int, _c_int, _c_int, _ptr, _ptr, _c_int, _c_f32, _ptr, _ptr, _c_int],
    'lnn_random_uniform_f32': [_c_int, _ptr, _c_u64, _c_u32, _c_f64, _c_f64],
    'lnn_random_normal_f32': [_c_int, _ptr, _c_u64, _c_u32, _c_f64, _c_f64],
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f'{LIB_PATH} not found: build it with `make -C litenn_amd/csrc` '
                           '(there is no CPU fallback)')
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _c_int
    lib.lnn_last_error.argtypes = []
    lib.lnn_last_error.restype = ctypes.c_char_p
    return lib


lib = _load()


def check(status):
    if status != OK:
        raise HipException(status, lib.lnn_last_error().decode('utf-8', 'replace'))


def _ints(seq):
    return (ctypes.c_int32 * len(seq))(*[int(x) for x in seq])


# ---- thin typed wrappers -------------------------------------------------
def device_count():
    n = _c_int(0)
    check(lib.lnn_device_count(ctypes.byref(n)))
    return n.value


def device_info(dev):
    name = ctypes.create_string_buffer(256)
    mem, cus, khz = _c_u64(0), _c_int(0), _c_int(0)
    check(lib.lnn_device_info(dev, name, 256, ctypes.byref(mem), ctypes.byref(cus), ctypes.byref(khz)))
    return dict(name=name.value.decode(), total_mem=mem.value, compute_units=cus.value, clock_khz=khz.value)


def release_device(dev):
    check(lib.lnn_release_device(dev))


def malloc(dev, nbytes):
    p = _ptr()
    check(lib.lnn_malloc(dev, nbytes, ctypes.byref(p)))
    return p.value


def free(dev, ptr):
    check(lib.lnn_free(dev, ptr))


def mem_info(dev):
    f, t = _c_u64(0), _c_u64(0)
    check(lib.lnn_mem_info(dev, ctypes.byref(f), ctypes.byref(t)))
    return f.value, t.value


def memcpy_h2d(dev, dst, array):
    check(lib.lnn_memcpy_h2d(dev, dst, array.ctypes.data, array.nbytes))


def memcpy_d2h(dev, array, src):
    check(lib.lnn_memcpy_d2h(dev, array.ctypes.data, src, array.nbytes))


def memcpy_d2d(dev, dst, src, nbytes):
    check(lib.lnn_memcpy_d2d(dev, dst, src, nbytes))


def fill_u32(dev, dst, pattern, count):
    check(lib.lnn_fill_u32(dev, dst, pattern, count))


def fill_f32(dev, dst, value, count):
    fill_u32(dev, dst, int(np.float32(value).view(np.uint32)), count)


def synchronize(dev):
    check(lib.lnn_synchronize(dev))


class Event:
    """hipEvent on the device's stream; Event.elapsed_ms(start, stop) waits for stop."""

    def __init__(self, dev):
        self.dev = dev
        p = _ptr()
        check(lib.lnn_event_create(dev, ctypes.byref(p)))
        self.handle = p.value

    def record(self):
        check(lib.lnn_event_record(self.dev, self.handle))
        return self

    @staticmethod
    def elapsed_ms(start, stop):
        ms = _c_f32(0)
        check(lib.lnn_event_elapsed_ms(start.dev, start.handle, stop.handle, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        if getattr(self, 'handle', None):
            lib.lnn_event_destroy(self.dev, self.handle)
            self.handle = None


def gemm(dev, trans_a, trans_b, batch, M, N, K, A, lda, sa, B, ldb, sb, C, ldc, sc, beta):
    check(lib.lnn_gemm_f32(dev, int(trans_a), int(trans_b), batch, M, N, K, A, lda, sa, B, ldb, sb, C, ldc, sc,
                           int(beta)))


def gemm_bias_act(dev, trans_a, trans_b, batch, M, N, K, A, lda, sa, B, ldb, sb, bias, act, slope, C, ldc, sc):
    """C = act(op(A) . op(B) + bias[n]); bias (N values, one per column of C) may be None; act as for
    conv2d_fwd_bias_act (ACT_NONE / ACT_LEAKY_RELU)."""
    check(lib.lnn_gemm_bias_act_f32(dev, int(trans_a), int(trans_b), batch, M, N, K, A, lda, sa, B, ldb, sb, bias,
                                    int(act), float(slope), C, ldc, sc))


def conv_desc(N, C, IH, IW, O, KH, KW, OH, OW, PADL, PADT, stride, dilation):
    return ConvDesc(N, C, IH, IW, O, KH, KW, OH, OW, PADL, PADT, stride, dilation)


def conv2d_fwd(dev, desc, X, W, Y, beta=0):
    check(lib.lnn_conv2d_fwd_f32(dev, ctypes.byref(desc), X, W, Y, int(beta)))


ACT_NONE, ACT_LEAKY_RELU = 0, 1


def conv2d_fwd_bias_act(dev, desc, X, W, bias, act, slope, Y):
    """Y = act(conv(X, W) + bias[o]); bias may be None."""
    check(lib.lnn_conv2d_fwd_bias_act_f32(dev, ctypes.byref(desc), X, W, bias, int(act), float(slope), Y))


def conv2d_dgrad(dev, desc, dY, W, dX, beta=1):
    check(lib.lnn_conv2d_dgrad_f32(dev, ctypes.byref(desc), dY, W, dX, int(beta)))


W_OIHW, W_IOHW = 0, 1
PASS_FWD, PASS_DGRAD, PASS_WGRAD = 0, 1, 2


def conv2d_weights_plan(desc, which):
    """True if the geometry's forward / data-gradient kernels read the permuted weights Wp[o][tap][c] (so the
    *_pw entry points apply), resp. if conv2d_wgrad_iohw serves its weight gradient.  Host arithmetic only."""
    yes = _c_int(0)
    check(lib.lnn_conv2d_weights_plan(ctypes.byref(desc), int(which), ctypes.byref(yes)))
    return bool(yes.value)


def conv2d_permute_weights(dev, desc, W, w_layout, Wp):
    check(lib.lnn_conv2d_permute_weights_f32(dev, ctypes.byref(desc), W, int(w_layout), Wp))


def conv2d_fwd_pw(dev, desc, X, Wp, bias, act, slope, Y, beta=0):
    check(lib.lnn_conv2d_fwd_pw_f32(dev, ctypes.byref(desc), X, Wp, bias, int(act), float(slope), Y, int(beta)))


def conv2d_dgrad_pw(dev, desc, dY, Wp, dX, beta=1):
    check(lib.lnn_conv2d_dgrad_pw_f32(dev, ctypes.byref(desc), dY, Wp, dX, int(beta)))


def conv2d_wgrad_iohw(dev, desc, X, dY, dW, beta=1):
    check(lib.lnn_conv2d_wgrad_iohw_f32(dev, ctypes.byref(desc), X, dY, dW, int(beta)))


NOALLOC_SCRATCH_BYTES = 32 << 20


def conv2d_wgrad_noalloc(dev, desc, X, dY, dW, beta=1):
    """conv2d_wgrad without device allocation: scratch is a fixed array inside the library (NOALLOC_SCRATCH_BYTES);
    problems that need more raise ERR_UNSUPPORTED."""
    check(lib.lnn_conv2d_wgrad_noalloc_f32(dev, ctypes.byref(desc), X, dY, dW, int(beta)))


FWD_PATH_IMPLICIT_GEMM, FWD_PATH_STEM_PATCH = 0, 1


def conv2d_wgrad_last_plan(dev):
    """(workgroups, K slices, equal runs across sub-tile borders?, tile rows) of the most recent weight gradient."""
    info = (ctypes.c_int32 * 4)()
    check(lib.lnn_conv2d_wgrad_last_plan(dev, info))
    return tuple(info)


def conv2d_fwd_path(desc, compute_units):
    """The kernel family conv2d_fwd picks for this geometry on a device with that many compute units (host
    arithmetic, needs no device)."""
    path = _c_int(-1)
    check(lib.lnn_conv2d_fwd_path(ctypes.byref(desc), int(compute_units), ctypes.byref(path)))
    return path.value


DGRAD_PATH_MFMA_TABLE, DGRAD_PATH_MFMA_TAP, DGRAD_PATH_VECTOR, DGRAD_PATH_STEM_MFMA = 0, 1, 2, 3


def conv2d_dgrad_path(desc, beta, compute_units):
    """(path, tile_info): the kernel family conv2d_dgrad picks for this geometry on a device with that many
    compute units, and for the vector-ALU path its tile extents (host arithmetic, needs no device)."""
    path = _c_int(-1)
    info = (ctypes.c_int32 * 7)()
    check(lib.lnn_conv2d_dgrad_path(ctypes.byref(desc), int(beta), int(compute_units), ctypes.byref(path), info))
    return path.value, dict(zip(('rows', 'cols', 'max_extent', 'min_row', 'min_col', 'max_row', 'max_col'), list(info)))


def conv2d_wgrad(dev, desc, X, dY, dW, beta=1):
    check(lib.lnn_conv2d_wgrad_f32(dev, ctypes.byref(desc), X, dY, dW, int(beta)))


def depthwise_conv2d_fwd(dev, desc, X, K, Y, beta=0):
    check(lib.lnn_depthwise_conv2d_fwd_f32(dev, ctypes.byref(desc), X, K, Y, int(beta)))


def depthwise_conv2d_dgrad(dev, desc, dY, K, dX, beta=1):
    check(lib.lnn_depthwise_conv2d_dgrad_f32(dev, ctypes.byref(desc), dY, K, dX, int(beta)))


def depthwise_conv2d_wgrad(dev, desc, X, dY, dK, beta=1):
    check(lib.lnn_depthwise_conv2d_wgrad_f32(dev, ctypes.byref(desc), X, dY, dK, int(beta)))


def unfold2d(dev, N, C, H, W, OH, OW, KH, KW, PADL, PADT, dilation, stride, order, is_transpose, src, dst, beta=0):
    check(lib.lnn_unfold2d_f32(dev, N, C, H, W, OH, OW, KH, KW, PADL, PADT, dilation, stride, order,
                               int(is_transpose), src, dst, int(beta)))


def transpose(dev, shape, axes, src, dst, beta=0):
    check(lib.lnn_transpose_f32(dev, len(shape), _ints(shape), _ints(axes), src, dst, int(beta)))


def ew_fwd(dev, op, n, src, dst, p0=0.0, beta=0):
    check(lib.lnn_ew_fwd_f32(dev, op, n, src, dst, float(p0), int(beta)))


def ew_bwd(dev, op, n, src, dout, din, p0=0.0, beta=1):
    check(lib.lnn_ew_bwd_f32(dev, op, n, src, dout, din, float(p0), beta))


def binary_bcast(dev, op, out_shape, a_shape, b_shape, a, b, out, beta=0):
    check(lib.lnn_binary_bcast_f32(dev, op, len(out_shape), _ints(out_shape), _ints(a_shape), _ints(b_shape),
                                   a, b, out, int(beta)))


def _mask(axes):
    m = 0
    for a in axes:
        m |= 1 << int(a)
    return m


def reduce_sum(dev, shape, axes, scale, src, dst, beta=0):
    check(lib.lnn_reduce_sum_f32(dev, len(shape), _ints(shape), _mask(axes), float(scale), src, dst, int(beta)))


def reduce_sum_bwd(dev, shape, axes, scale, dout, din, beta=1):
    check(lib.lnn_reduce_sum_bwd_f32(dev, len(shape), _ints(shape), _mask(axes), float(scale), dout, din, beta))


def sgd_update(dev, n, v, g, acc, momentum, lr, nesterov):
    check(lib.lnn_sgd_update_f32(dev, n, v, g, acc, float(momentum), float(lr), int(bool(nesterov))))


def adam_update(dev, n, t, g, m, v, beta1, beta2, lr):
    check(lib.lnn_adam_update_f32(dev, int(n), t, g, m, v, float(beta1), float(beta2), float(lr)))


def random_uniform(dev, out, n, seed, low, high):
    check(lib.lnn_random_uniform_f32(dev, out, int(n), int(seed), float(low), float(high)))


def random_normal(dev, out, n, seed, mean, stddev):
    check(lib.lnn_random_normal_f32(dev, out, int(n), int(seed), float(mean), float(stddev)))


def bias_act_bwd(dev, N, O, HW, y, dy, act, slope, dpre, dbias, beta_bias):
    check(lib.lnn_bias_act_bwd_f32(dev, N, O, HW, y, dy, act, float(slope), dpre, dbias, beta_bias))


def _ptr_array(ptrs):
    return (ctypes.c_void_p * len(ptrs))(*ptrs)


def sgd_update_multi(dev, ns, vs, gs, accs, momentum, lr, nesterov):
    """One launch for the SGD update of len(ns) tensors."""
    count = len(ns)
    check(lib.lnn_sgd_update_multi_f32(dev, count, (ctypes.c_uint64 * count)(*ns), _ptr_array(vs), _ptr_array(gs),
                                       _ptr_array(accs), float(momentum), float(lr), 1 if nesterov else 0))


def sgd_update_multi_wp(dev, ns, vs, gs, accs, momentum, lr, nesterov, wps, cs, kks, layouts=None):
    """sgd_update_multi that also stores the new values in the tensors' permuted copies Wp[o][tap][c] (wps[i] a device
    pointer or None, cs[i] / kks[i] the copy's C and KH*KW, layouts[i] W_OIHW / W_IOHW: how tensor i is stored)."""
    count = len(ns)
    lay = (ctypes.c_int32 * count)(*layouts) if layouts is not None else None
    check(lib.lnn_sgd_update_multi_wp_f32(dev, count, (ctypes.c_uint64 * count)(*ns), _ptr_array(vs), _ptr_array(gs),
                                          _ptr_array(accs), float(momentum), float(lr), 1 if nesterov else 0,
                                          _ptr_array(wps), (ctypes.c_int32 * count)(*cs), (ctypes.c_int32 * count)(*kks), lay))


def adam_update_multi_wp(dev, ns, ts, gs, ms, vs, beta1, beta2, lr, wps, cs, kks, layouts=None):
    """adam_update_multi that also stores the new values in the tensors' permuted copies (see sgd_update_multi_wp)."""
    count = len(ns)
    lay = (ctypes.c_int32 * count)(*layouts) if layouts is not None else None
    check(lib.lnn_adam_update_multi_wp_f32(dev, count, (ctypes.c_uint64 * count)(*ns), _ptr_array(ts), _ptr_array(gs),
                                           _ptr_array(ms), _ptr_array(vs), float(beta1), float(beta2), float(lr),
                                           _ptr_array(wps), (ctypes.c_int32 * count)(*cs), (ctypes.c_int32 * count)(*kks), lay))


def _wp_arrays(count, wps, cs, kks, layouts):
    if wps is None:
        return None, None, None, None
    lay = (ctypes.c_int32 * count)(*layouts) if layouts is not None else None
    return _ptr_array(wps), (ctypes.c_int32 * count)(*cs), (ctypes.c_int32 * count)(*kks), lay


def sgd_update_multi_lrd(dev, ns, vs, gs, accs, momentum, lr, nesterov, lr_dropout, seeds, wps=None, cs=None, kks=None,
                         layouts=None):
    """sgd_update_multi(_wp) with learning-rate dropout: seeds holds two uint32 per tensor (accumulator kernel, value
    kernel), as the reference draws them (Optimizer.py:178-182)."""
    count = len(ns)
    check(lib.lnn_sgd_update_multi_lrd_f32(dev, count, (ctypes.c_uint64 * count)(*ns), _ptr_array(vs), _ptr_array(gs),
                                           _ptr_array(accs), float(momentum), float(lr), 1 if nesterov else 0,
                                           float(lr_dropout), (ctypes.c_uint32 * (2 * count))(*seeds),
                                           *_wp_arrays(count, wps, cs, kks, layouts)))


def adam_update_multi_lrd(dev, ns, ts, gs, ms, vs, beta1, beta2, lr, lr_dropout, seeds, wps=None, cs=None, kks=None,
                          layouts=None):
    """adam_update_multi(_wp) with learning-rate dropout: one uint32 seed per tensor."""
    count = len(ns)
    check(lib.lnn_adam_update_multi_lrd_f32(dev, count, (ctypes.c_uint64 * count)(*ns), _ptr_array(ts), _ptr_array(gs),
                                            _ptr_array(ms), _ptr_array(vs), float(beta1), float(beta2), float(lr),
                                            float(lr_dropout), (ctypes.c_uint32 * count)(*seeds),
                                            *_wp_arrays(count, wps, cs, kks, layouts)))


def adam_update_multi(dev, ns, ts, gs, ms, vs, beta1, beta2, lr):
    """One launch for the Adam update of len(ns) tensors."""
    count = len(ns)
    check(lib.lnn_adam_update_multi_f32(dev, count, (ctypes.c_uint64 * count)(*ns), _ptr_array(ts), _ptr_array(gs),
                                        _ptr_array(ms), _ptr_array(vs), float(beta1), float(beta2), float(lr)))
