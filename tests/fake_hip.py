"""A numpy stand-in for the C ABI binding, for host-logic tests without a GPU.

TEST CODE ONLY.  It is patched over `litenn_amd.core.hip.api` by the
`nn_backend` fixture so that Tensor / autograd / buffer-pool / module logic can
be exercised on the CPU; the arithmetic comes from the oracle.  The shipped
package has no such path: without liblitenn_hip.so and a GPU it raises.
"""
import numpy as np

from oracle import (conv2d_fwd, conv2d_dx, conv2d_dw, unfold_index_map, unfold_T_index_map, apply_index_map,
                    depthwise_fwd, depthwise_di, depthwise_dk)
from litenn_amd.core.hip import api as real_api

NAMES = ['device_count', 'device_info', 'release_device', 'malloc', 'free', 'mem_info', 'memcpy_h2d', 'memcpy_d2h',
         'memcpy_d2d', 'fill_u32', 'fill_f32', 'synchronize', 'gemm', 'gemm_bias_act', 'conv2d_fwd', 'conv2d_fwd_bias_act', 'conv2d_dgrad', 'conv2d_wgrad', 'conv2d_permute_weights', 'conv2d_fwd_pw', 'conv2d_dgrad_pw', 'conv2d_wgrad_iohw', 'depthwise_conv2d_fwd', 'depthwise_conv2d_dgrad', 'depthwise_conv2d_wgrad',
         'unfold2d', 'transpose', 'ew_fwd', 'ew_bwd', 'binary_bcast', 'reduce_sum', 'reduce_sum_bwd', 'sgd_update', 'adam_update', 'random_uniform', 'random_normal', 'bias_act_bwd', 'sgd_update_multi', 'sgd_update_multi_wp', 'adam_update_multi_wp', 'adam_update_multi', 'sgd_update_multi_lrd', 'adam_update_multi_lrd']


class FakeHip:
    def __init__(self, capacity=None):
        self.mem = {}
        self.next_ptr = 0x10000
        self.capacity = capacity
        self.launches = 0
        self.mallocs = 0

    # -- memory
    def used(self):
        return sum(a.nbytes for a in self.mem.values())

    def device_count(self): return 1
    def device_info(self, dev): return dict(name='fake-hip', total_mem=1 << 34, compute_units=4, clock_khz=1000)
    def release_device(self, dev): pass
    def mem_info(self, dev): return (1 << 34) - self.used(), 1 << 34
    def synchronize(self, dev): pass

    def malloc(self, dev, nbytes):
        if self.capacity is not None and self.used() + nbytes > self.capacity:
            raise real_api.HipException(real_api.ERR_OOM, 'fake out of memory')
        ptr = self.next_ptr
        self.next_ptr += (nbytes + 0xfff) & ~0xfff
        # NaN-filled: a read of memory nobody initialised poisons the result
        self.mem[ptr] = np.full((nbytes + 3) // 4, np.nan, np.float32)
        self.mallocs += 1
        return ptr

    def free(self, dev, ptr):
        del self.mem[ptr]

    def f(self, ptr, shape=None):
        a = self.mem[ptr]
        return a if shape is None else a[:int(np.prod(shape))].reshape(shape)

    def memcpy_h2d(self, dev, dst, array):
        self.f(dst)[:array.size] = np.asarray(array, np.float32).reshape(-1)

    def memcpy_d2h(self, dev, array, src):
        array.reshape(-1)[:] = self.f(src)[:array.size]

    def memcpy_d2d(self, dev, dst, src, nbytes):
        self.f(dst)[:nbytes // 4] = self.f(src)[:nbytes // 4]

    def fill_u32(self, dev, dst, pattern, count):
        self.f(dst).view(np.uint32)[:count] = np.uint32(pattern)

    def fill_f32(self, dev, dst, value, count):
        self.f(dst)[:count] = np.float32(value)

    @staticmethod
    def _put(out, val, beta):
        val = np.asarray(val, np.float64)
        out[...] = (out.astype(np.float64) + val if beta else val).astype(np.float32)

    # -- contraction kernels
    def gemm(self, dev, ta, tb, batch, M, N, K, A, lda, sa, B, ldb, sb, C, ldc, sc, beta):
        self.launches += 1
        assert lda == (M if ta else K) and ldb == (K if tb else N) and ldc == N, 'fake gemm: dense operands only'
        a = self.f(A, (batch, K, M) if ta else (batch, M, K)).astype(np.float64)
        b = self.f(B, (batch, N, K) if tb else (batch, K, N)).astype(np.float64)
        r = np.matmul(a.transpose(0, 2, 1) if ta else a, b.transpose(0, 2, 1) if tb else b)
        self._put(self.f(C, (batch, M, N)), r, beta)

    def gemm_bias_act(self, dev, ta, tb, batch, M, N, K, A, lda, sa, B, ldb, sb, bias, act, slope, C, ldc, sc):
        self.launches += 1
        assert lda == (M if ta else K) and ldb == (K if tb else N) and ldc == N, 'fake gemm: dense operands only'
        a = self.f(A, (batch, K, M) if ta else (batch, M, K)).astype(np.float64)
        b = self.f(B, (batch, N, K) if tb else (batch, K, N)).astype(np.float64)
        r = np.matmul(a.transpose(0, 2, 1) if ta else a, b.transpose(0, 2, 1) if tb else b).astype(np.float32)
        if bias is not None:
            r = r + self.f(bias, (N,)).reshape(1, 1, -1)
        if act == 1:
            r = np.where(r >= 0, r, np.float32(slope) * r)
        self._put(self.f(C, (batch, M, N)), r, 0)

    @staticmethod
    def _geom(d):
        xs = (d.N, d.C, d.IH, d.IW)
        ws = (d.O, d.C, d.KH, d.KW)
        ys = (d.N, d.O, d.OH, d.OW)
        # the oracle derives OH/OW itself from a (left, top, right, bottom) tuple that reproduces them
        pr = (d.OW - 1) * d.stride + (d.KW - 1) * d.dilation + 1 - d.IW - d.PADL
        pb = (d.OH - 1) * d.stride + (d.KH - 1) * d.dilation + 1 - d.IH - d.PADT
        return xs, ws, ys, (d.PADL, d.PADT, max(pr, 0), max(pb, 0))

    def conv2d_fwd(self, dev, d, X, W, Y, beta=0):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        r = conv2d_fwd(self.f(X, xs), self.f(W, ws), d.stride, d.dilation, pad)
        assert r.shape == ys, (r.shape, ys)
        self._put(self.f(Y, ys), r, beta)

    def conv2d_fwd_bias_act(self, dev, d, X, W, bias, act, slope, Y):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        r = conv2d_fwd(self.f(X, xs), self.f(W, ws), d.stride, d.dilation, pad).astype(np.float32)
        if bias is not None:
            r = r + self.f(bias, (d.O,)).reshape(1, -1, 1, 1)
        if act == 1:
            r = np.where(r >= 0, r, np.float32(slope) * r)
        self._put(self.f(Y, ys), r, 0)

    def conv2d_dgrad(self, dev, d, dY, W, dX, beta=1):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        self._put(self.f(dX, xs), conv2d_dx(self.f(dY, ys), self.f(W, ws), xs, d.stride, d.dilation, pad), beta)

    def conv2d_wgrad(self, dev, d, X, dY, dW, beta=1):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        self._put(self.f(dW, ws), conv2d_dw(self.f(X, xs), self.f(dY, ys), ws, d.stride, d.dilation, pad), beta)

    # the weights in the kernels' permuted layout Wp[o][tap][c]
    def conv2d_permute_weights(self, dev, d, W, w_layout, Wp):
        self.launches += 1
        kk = d.KH * d.KW
        if w_layout == real_api.W_OIHW:
            w = self.f(W, (d.O, d.C, kk))
        else:
            w = self.f(W, (d.C, d.O, kk)).transpose(1, 0, 2)
        self.f(Wp, (d.O, kk, d.C))[...] = w.transpose(0, 2, 1)

    def _from_wp(self, d, Wp):
        assert real_api.conv2d_weights_plan(d, real_api.PASS_FWD) or real_api.conv2d_weights_plan(d, real_api.PASS_DGRAD)
        return np.ascontiguousarray(self.f(Wp, (d.O, d.KH * d.KW, d.C)).transpose(0, 2, 1)).reshape(d.O, d.C, d.KH, d.KW)

    def conv2d_fwd_pw(self, dev, d, X, Wp, bias, act, slope, Y, beta=0):
        self.launches += 1
        assert real_api.conv2d_weights_plan(d, real_api.PASS_FWD), 'forward of this geometry does not read permuted weights'
        xs, ws, ys, pad = self._geom(d)
        r = conv2d_fwd(self.f(X, xs), self._from_wp(d, Wp), d.stride, d.dilation, pad)
        if bias is not None or act:
            assert not beta
            r = r.astype(np.float32)
            if bias is not None:
                r = r + self.f(bias, (d.O,)).reshape(1, -1, 1, 1)
            if act == 1:
                r = np.where(r >= 0, r, np.float32(slope) * r)
        self._put(self.f(Y, ys), r, beta)

    def conv2d_dgrad_pw(self, dev, d, dY, Wp, dX, beta=1):
        self.launches += 1
        assert real_api.conv2d_weights_plan(d, real_api.PASS_DGRAD), 'dgrad of this geometry does not read permuted weights'
        xs, ws, ys, pad = self._geom(d)
        self._put(self.f(dX, xs), conv2d_dx(self.f(dY, ys), self._from_wp(d, Wp), xs, d.stride, d.dilation, pad), beta)

    def conv2d_wgrad_iohw(self, dev, d, X, dY, dW, beta=1):
        self.launches += 1
        assert real_api.conv2d_weights_plan(d, real_api.PASS_WGRAD), 'wgrad of this geometry cannot write swapped axes'
        xs, ws, ys, pad = self._geom(d)
        dw = conv2d_dw(self.f(X, xs), self.f(dY, ys), ws, d.stride, d.dilation, pad)
        self._put(self.f(dW, (d.C, d.O, d.KH, d.KW)), dw.transpose(1, 0, 2, 3), beta)

    def depthwise_conv2d_fwd(self, dev, d, X, K, Y, beta=0):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        self._put(self.f(Y, ys), depthwise_fwd(self.f(X, xs), self.f(K, (d.C, d.KH, d.KW)), d.stride, d.dilation, pad), beta)

    def depthwise_conv2d_dgrad(self, dev, d, dY, K, dX, beta=1):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        self._put(self.f(dX, xs), depthwise_di(self.f(dY, ys), self.f(K, (d.C, d.KH, d.KW)), xs, d.stride, d.dilation, pad), beta)

    def depthwise_conv2d_wgrad(self, dev, d, X, dY, dK, beta=1):
        self.launches += 1
        xs, ws, ys, pad = self._geom(d)
        ks = (d.C, d.KH, d.KW)
        self._put(self.f(dK, ks), depthwise_dk(self.f(X, xs), self.f(dY, ys), ks, d.stride, d.dilation, pad), beta)

    def unfold2d(self, dev, N, C, H, W, OH, OW, KH, KW, PADL, PADT, dil, stride, order, is_transpose, src, dst, beta=0):
        self.launches += 1
        fn = unfold_T_index_map if is_transpose else unfold_index_map
        shape, m = fn(N, C, H, W, OH, OW, KH, KW, PADL, PADT, dil, stride, ('CJI_NHW', 'NHW_CJI')[order])
        self._put(self.f(dst, shape), apply_index_map(self.f(src, (N * C * H * W,)), shape, m), beta)

    def transpose(self, dev, shape, axes, src, dst, beta=0):
        self.launches += 1
        r = self.f(src, shape).transpose(axes)
        self._put(self.f(dst, r.shape), r, beta)

    # -- pointwise / reductions
    _F = {0: lambda x, p: x + p, 1: lambda x, p: x * p, 2: lambda x, p: np.where(x >= 0, x, p * x),
          3: lambda x, p: x * x, 4: lambda x, p: np.where(x >= 0, x, 0)}
    _DF = {0: lambda x, p: np.ones_like(x), 1: lambda x, p: np.full_like(x, p), 2: lambda x, p: np.where(x >= 0, 1, p),
           3: lambda x, p: 2 * x, 4: lambda x, p: np.where(x >= 0, 1.0, 0.0)}

    def ew_fwd(self, dev, op, n, src, dst, p0=0.0, beta=0):
        self.launches += 1
        x = self.f(src)[:n].astype(np.float64)
        self._put(self.f(dst)[:n], self._F[op](x, p0), beta)

    def ew_bwd(self, dev, op, n, src, dout, din, p0=0.0, beta=1):
        self.launches += 1
        x = self.f(src)[:n].astype(np.float64)
        self._put(self.f(din)[:n], self.f(dout)[:n].astype(np.float64) * self._DF[op](x, p0), beta)

    def binary_bcast(self, dev, op, out_shape, a_shape, b_shape, a, b, out, beta=0):
        self.launches += 1
        x, y = self.f(a, a_shape).astype(np.float64), self.f(b, b_shape).astype(np.float64)
        self._put(self.f(out, out_shape), (x + y, x - y, x * y)[op], beta)

    def reduce_sum(self, dev, shape, axes, scale, src, dst, beta=0):
        self.launches += 1
        r = self.f(src, shape).astype(np.float64).sum(axis=tuple(axes)) * scale if len(axes) else \
            self.f(src, shape).astype(np.float64) * scale
        r = np.asarray(r).reshape(-1)
        self._put(self.f(dst)[:r.size], r, beta)

    def reduce_sum_bwd(self, dev, shape, axes, scale, dout, din, beta=1):
        self.launches += 1
        kd = tuple(1 if i in axes else s for i, s in enumerate(shape))
        g = self.f(dout, kd).astype(np.float64) * scale
        self._put(self.f(din, shape), np.broadcast_to(g, shape), beta)

    def sgd_update(self, dev, n, v, g, acc, momentum, lr, nesterov):
        self.launches += 1
        V, G, A = self.f(v)[:n], self.f(g)[:n], self.f(acc)[:n]
        a = (np.float32(momentum) * A - np.float32(lr) * G).astype(np.float32)
        A[:] = a
        V[:] = V + ((np.float32(momentum) * a - np.float32(lr) * G) if nesterov else a)

    def adam_update(self, dev, n, t, g, m, v, beta1, beta2, lr):
        self.launches += 1
        T, G, M, V = self.f(t)[:n], self.f(g)[:n], self.f(m)[:n], self.f(v)[:n]
        b1, b2 = np.float32(beta1), np.float32(beta2)
        M[:] = b1 * M + (np.float32(1) - b1) * G
        V[:] = b2 * V + (np.float32(1) - b2) * G * G
        T[:] = T - np.float32(lr) * M / (np.sqrt(V) + np.float32(1e-7))

    def sgd_update_multi(self, dev, ns, vs, gs, accs, momentum, lr, nesterov):
        for n, v, g, a in zip(ns, vs, gs, accs):
            self.sgd_update(dev, n, v, g, a, momentum, lr, nesterov)
        self.launches -= len(ns) - 1

    def _refresh_copies(self, ns, vs, wps, cs, kks, layouts):
        for i, (n, v, wp, c, kk) in enumerate(zip(ns, vs, wps, cs, kks)):
            if wp is not None and n:
                o = n // (c * kk)
                if layouts is not None and layouts[i] == real_api.W_IOHW:
                    self.f(wp, (o, kk, c))[...] = self.f(v, (c, o, kk)).transpose(1, 2, 0)
                else:
                    self.f(wp, (o, kk, c))[...] = self.f(v, (o, c, kk)).transpose(0, 2, 1)

    def sgd_update_multi_wp(self, dev, ns, vs, gs, accs, momentum, lr, nesterov, wps, cs, kks, layouts=None):
        self.sgd_update_multi(dev, ns, vs, gs, accs, momentum, lr, nesterov)
        self._refresh_copies(ns, vs, wps, cs, kks, layouts)

    def adam_update_multi_wp(self, dev, ns, ts, gs, ms, vs, beta1, beta2, lr, wps, cs, kks, layouts=None):
        self.adam_update_multi(dev, ns, ts, gs, ms, vs, beta1, beta2, lr)
        self._refresh_copies(ns, ts, wps, cs, kks, layouts)

    def adam_update_multi(self, dev, ns, ts, gs, ms, vs, beta1, beta2, lr):
        for n, t, g, m, v in zip(ns, ts, gs, ms, vs):
            self.adam_update(dev, n, t, g, m, v, beta1, beta2, lr)
        self.launches -= len(ns) - 1

    def sgd_update_multi_lrd(self, dev, ns, vs, gs, accs, momentum, lr, nesterov, lr_dropout, seeds, wps=None, cs=None,
                             kks=None, layouts=None):
        from oracle import hash_rng
        self.launches += 1
        mom, lr32 = np.float32(momentum), np.float32(lr)
        for i, (n, v, g, acc) in enumerate(zip(ns, vs, gs, accs)):
            V, G, A = self.f(v)[:n], self.f(g)[:n], self.f(acc)[:n]
            lr_a = np.where(hash_rng.lr_dropout_mask(n, seeds[2 * i], lr_dropout), np.float32(0), lr32) if lr_dropout else lr32
            lr_t = np.where(hash_rng.lr_dropout_mask(n, seeds[2 * i + 1], lr_dropout), np.float32(0), lr32) if lr_dropout else lr32
            a = (mom * A - lr_a * G).astype(np.float32)
            A[:] = a
            V[:] = V + ((mom * a - lr_t * G) if nesterov else a)
        if wps is not None:
            self._refresh_copies(ns, vs, wps, cs, kks, layouts)

    def adam_update_multi_lrd(self, dev, ns, ts, gs, ms, vs, beta1, beta2, lr, lr_dropout, seeds, wps=None, cs=None,
                              kks=None, layouts=None):
        from oracle import hash_rng
        self.launches += 1
        b1, b2, lr32 = np.float32(beta1), np.float32(beta2), np.float32(lr)
        for i, (n, t, g, m, v) in enumerate(zip(ns, ts, gs, ms, vs)):
            T, G, M, V = self.f(t)[:n], self.f(g)[:n], self.f(m)[:n], self.f(v)[:n]
            lr_t = np.where(hash_rng.lr_dropout_mask(n, seeds[i], lr_dropout), np.float32(0), lr32) if lr_dropout else lr32
            M[:] = b1 * M + (np.float32(1) - b1) * G
            V[:] = b2 * V + (np.float32(1) - b2) * G * G
            T[:] = T - lr_t * M / (np.sqrt(V) + np.float32(1e-7))
        if wps is not None:
            self._refresh_copies(ns, ts, wps, cs, kks, layouts)

    def bias_act_bwd(self, dev, N, O, HW, y, dy, act, slope, dpre, dbias, beta_bias):
        self.launches += 1
        n = N * O * HW
        g = self.f(dy)[:n].copy()
        if act == real_api.ACT_LEAKY_RELU:
            g *= np.where(self.f(y)[:n] >= 0, np.float32(1), np.float32(slope))
        if dpre is not None:
            self.f(dpre)[:n] = g
        if dbias is not None:
            db = g.reshape(N, O, HW).astype(np.float64).sum(axis=(0, 2)).astype(np.float32)
            B = self.f(dbias)[:O]
            B[:] = B + db if beta_bias else db

    def random_uniform(self, dev, out, n, seed, low, high):
        from oracle import hash_rng
        self.launches += 1
        self.f(out)[:n] = hash_rng.random_uniform(n, seed, low, high)

    def random_normal(self, dev, out, n, seed, mean, stddev):
        from oracle import hash_rng
        self.launches += 1
        self.f(out)[:n] = hash_rng.random_normal(n, seed, mean, stddev)


def install(monkeypatch, capacity=None):
    fake = FakeHip(capacity)
    for name in NAMES:
        monkeypatch.setattr(real_api, name, getattr(fake, name))
    return fake
