"""ctypes front end of the C restatement of the reference path (refpath.c).

TEST INFRASTRUCTURE ONLY (second checker with the reference's fp32 summation
order, and the timed CPU baseline of the benchmark).  Build with
`make -C oracle`; the shared object lands in oracle/_build/.
"""
import ctypes
import os
import subprocess

import numpy as np

from .conv_info import info_conv2d

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, '_build', 'librefpath.so')
_lib = None

_f32p = np.ctypeslib.ndpointer(np.float32, flags='C_CONTIGUOUS')
_i32p = np.ctypeslib.ndpointer(np.int32, flags='C_CONTIGUOUS')
_I = ctypes.c_int


def build(force=False):
    """Compile refpath.c (gcc, OpenMP).  Returns the path of the .so."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(['make', '-C', _HERE] + (['-B'] if force else []),
                              stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.ref_num_threads.restype = _I
        L.ref_unfold2d.argtypes = [_f32p, _f32p] + [_I] * 15
        L.ref_unfold2d.restype = None
        L.ref_transpose.argtypes = [_f32p, _f32p, _I, _i32p, _i32p, _I]
        L.ref_transpose.restype = None
        L.ref_matmul.argtypes = [_f32p, _f32p, _f32p] + [_I] * 5
        L.ref_matmul.restype = None
        L.ref_matmul_bwd.argtypes = [_f32p] * 5 + [_I] * 4
        L.ref_matmul_bwd.restype = _I
        L.ref_gemm_tile_widths.argtypes = [_I, _I, _I, ctypes.POINTER(_I), ctypes.POINTER(_I)]
        L.ref_gemm_tile_widths.restype = None
        for name in ('ref_conv2d_fwd', 'ref_conv2d_dx', 'ref_conv2d_dw'):
            fn = getattr(L, name)
            fn.argtypes = [_f32p] * 3 + [_I] * 13
            fn.restype = _I
        _lib = L
    return _lib


def num_threads():
    return int(lib().ref_num_threads())


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _geom(x_shape, w_shape, stride, dilation, padding):
    N, C, IH, IW = x_shape
    O, KI, KH, KW = w_shape
    if KI != C:
        raise ValueError('channel mismatch')
    ci = info_conv2d(IH, IW, KH, KW, stride, dilation, padding)
    return (N, C, IH, IW, O, KH, KW, ci.OH, ci.OW, ci.PADL, ci.PADT, stride, dilation)


def conv2d_fwd(x, w, stride=1, dilation=1, padding='same'):
    g = _geom(x.shape, w.shape, stride, dilation, padding)
    y = np.empty((g[0], g[4], g[7], g[8]), np.float32)
    if lib().ref_conv2d_fwd(_f32(x), _f32(w), y, *g) != 0:
        raise MemoryError('refpath: allocation failed')
    return y


def conv2d_dx(dy, w, x_shape, stride=1, dilation=1, padding='same', into=None):
    g = _geom(x_shape, w.shape, stride, dilation, padding)
    dx = np.zeros(x_shape, np.float32) if into is None else into
    if lib().ref_conv2d_dx(_f32(dy), _f32(w), dx, *g) != 0:
        raise MemoryError('refpath: allocation failed')
    return dx


def conv2d_dw(x, dy, w_shape, stride=1, dilation=1, padding='same', into=None):
    g = _geom(x.shape, w_shape, stride, dilation, padding)
    dw = np.zeros(w_shape, np.float32) if into is None else into
    if lib().ref_conv2d_dw(_f32(x), _f32(dy), dw, *g) != 0:
        raise MemoryError('refpath: allocation failed')
    return dw


def matmul(a, b, into=None, add=False):
    M, K = a.shape[-2:]
    N = b.shape[-1]
    batch = int(np.prod(a.shape[:-2], dtype=np.int64))
    c = np.zeros(b.shape[:-2] + (M, N), np.float32) if into is None else into
    lib().ref_matmul(_f32(a), _f32(b), c, batch, M, K, N, int(add))
    return c


def matmul_bwd(a, b, dc, da=None, db=None):
    M, K = a.shape[-2:]
    N = b.shape[-1]
    batch = int(np.prod(a.shape[:-2], dtype=np.int64))
    da = np.zeros(a.shape, np.float32) if da is None else da
    db = np.zeros(b.shape, np.float32) if db is None else db
    if lib().ref_matmul_bwd(_f32(a), _f32(b), _f32(dc), da, db, batch, M, K, N) != 0:
        raise MemoryError('refpath: allocation failed')
    return da, db


def gemm_tile_widths(M, N, K):
    mw, kw = _I(1), _I(1)
    lib().ref_gemm_tile_widths(M, N, K, ctypes.byref(mw), ctypes.byref(kw))
    return mw.value, kw.value


def unfold2d(x, N, C, H, W, OH, OW, KH, KW, PADL, PADT, DIL, STRIDE, order, is_transpose):
    out = np.empty(N * C * OH * OW * KH * KW, np.float32)
    lib().ref_unfold2d(out, _f32(x), N, C, H, W, OH, OW, KH, KW, PADL, PADT, DIL, STRIDE,
                       order, int(is_transpose), 0)
    return out


def transpose(x, axes):
    x = _f32(x)
    out = np.empty(tuple(x.shape[a] for a in axes), np.float32)
    lib().ref_transpose(out, x, x.ndim, np.asarray(x.shape, np.int32), np.asarray(axes, np.int32), 0)
    return out
