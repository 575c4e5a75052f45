#!/usr/bin/env python3
"""Benchmark of the conv2D / matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--all] [--config NAME]

Default workload (the configuration the headline metric is quoted on): the
VGG-style 3x3 convolution layer, fp32 NCHW, N=32, C=128, H=W=56, O=128,
stride 1, padding 'same'.  One step = forward + dX + dW (gradients accumulate
into their buffers, as the reference's backward does), inputs resident in HBM.
Prints ONE JSON line: whole-step TFLOP/s, the fp32-MFMA roofline fraction of
the dominant kernel (timed with HIP events on the library's stream), and the
CPU restatement of the reference algorithm timed on the host cores.

--all additionally measures every benchmark configuration (conv geometries,
the 4096^3 matmul with both gradients, the 4-layer encoder training step) and
writes one JSON object per line to bench_all.jsonl in --out-dir (default: the current directory).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # 256 CU x 2.4 GHz x 256 flop/clk/CU
PEAK_HBM_GBS = 8000.0

def measured_traffic():
    """HBM bytes per launch from hardware counters (FETCH_SIZE + WRITE_SIZE, each scaled by its reading for a plain
    copy of known size), measured separately under rocprofv3 --pmc: the `traffic_bytes <workload> <pass> <bytes>`
    lines of the committed summaries profiles/*_hbm_traffic_pmc.txt.  A pass that has not been measured reports null."""
    import glob
    table = {}
    for path in sorted(glob.glob(os.path.join(ROOT, 'profiles', '*_hbm_traffic_pmc.txt'))):
        for line in open(path):
            f = line.split()
            if len(f) == 4 and f[0] == 'traffic_bytes':
                table.setdefault(f[1], {})[f[2]] = float(f[3])
    return table


MEASURED_TRAFFIC_BYTES = measured_traffic()

CONV_CONFIGS = {
    # name: (x shape, w shape, stride, dilation, padding, seed)
    'cfg1_stem3x3': ((8, 3, 64, 64), (32, 3, 3, 3), 1, 1, 'same', 0),
    'cfg3_vgg3x3': ((32, 128, 56, 56), (128, 128, 3, 3), 1, 1, 'same', 0),
    'cfg4a_stem7x7s2': ((32, 3, 224, 224), (64, 3, 7, 7), 2, 1, 3, 0),
    'cfg4b_pointwise': ((64, 256, 28, 28), (512, 256, 1, 1), 1, 1, 'same', 1),
    'cfg4c_dilated': ((16, 64, 64, 64), (64, 64, 3, 3), 1, 2, 2, 2),
}


def conv_info(xs, ws, s, d, padding):
    from litenn_amd.core.info import InfoConv2D
    return InfoConv2D(xs[2], xs[3], ws[2], ws[3], s, d, padding)


def conv_tensors(xs, ws, s, d, padding, seed):
    rs = np.random.RandomState(seed)
    x = rs.uniform(-1, 1, xs).astype(np.float32)
    w = rs.normal(0, np.sqrt(2.0 / (ws[1] * ws[2] * ws[3])), ws).astype(np.float32)
    ci = conv_info(xs, ws, s, d, padding)
    dy = rs.normal(0, 1, (xs[0], ws[0], ci.OH, ci.OW)).astype(np.float32)
    return x, w, dy, ci


class Dev:
    """Device array helper over the C ABI."""

    def __init__(self, api, array=None, shape=None):
        self.api = api
        if array is not None:
            shape = array.shape
        self.shape = tuple(shape)
        self.count = int(np.prod(self.shape, dtype=np.int64))
        self.ptr = api.malloc(0, self.count * 4)
        if array is not None:
            api.memcpy_h2d(0, self.ptr, np.ascontiguousarray(array, dtype=np.float32))
        else:
            api.fill_f32(0, self.ptr, 0.0, self.count)

    def get(self):
        out = np.empty(self.shape, np.float32)
        self.api.memcpy_d2h(0, out, self.ptr)
        return out

    def zero(self):
        self.api.fill_f32(0, self.ptr, 0.0, self.count)

    def free(self):
        self.api.free(0, self.ptr)


def time_events(api, fn, iters):
    """Average milliseconds of fn() over `iters` back-to-back launches, from
    HIP events recorded on the stream the kernels run on."""
    e0, e1 = api.Event(0), api.Event(0)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    return api.Event.elapsed_ms(e0, e1) / iters


class InStepTimer:
    """Durations of chosen library calls where their caller sees them: inside a whole step, between the launches that
    precede and follow them there (cold caches, whatever the previous pass left in the memory-side cache), instead of
    the same pass launched back to back.  Wraps functions of the binding module by name; every wrapped call is
    bracketed by two HIP events on the library's stream.  label(args) names the call (e.g. by layer)."""

    def __init__(self, api, names, label=None):
        self.api, self.names, self.label = api, names, label or (lambda name, args: name)
        self.saved, self.records, self.pool = {}, [], []

    def __enter__(self):
        for name in self.names:
            orig = getattr(self.api, name)
            self.saved[name] = orig

            def wrapped(*args, _orig=orig, _name=name):
                e0 = self.pool.pop() if self.pool else self.api.Event(0)
                e1 = self.pool.pop() if self.pool else self.api.Event(0)
                e0.record()
                _orig(*args)
                e1.record()
                self.records.append((self.label(_name, args), e0, e1))
            setattr(self.api, name, wrapped)
        return self

    def __exit__(self, *exc):
        for name, orig in self.saved.items():
            setattr(self.api, name, orig)

    def per_step_ms(self, steps):
        """{label: milliseconds per step}, summed over the calls that share a label."""
        out = {}
        for label, e0, e1 in self.records:
            out[label] = out.get(label, 0.0) + self.api.Event.elapsed_ms(e0, e1)
            self.pool += [e0, e1]
        self.records = []
        return {k: v / steps for k, v in out.items()}


def launch_floor_ms(api):
    """What the box charges for any launch through the library: a one-word fill (a kernel with nothing to do), launched
    back to back and timed like the passes, with HIP events on the library's stream."""
    tiny = Dev(api, shape=(64,))
    for _ in range(50):
        api.fill_u32(0, tiny.ptr, 0, 1)
    ms = min(time_events(api, lambda: api.fill_u32(0, tiny.ptr, 0, 1), 300) for _ in range(3))
    tiny.free()
    return ms


def rel_err(got, ref):
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


SETTLE_S = 0.25
CPU_OPENCL = 'not probed'


def settle(step, sync):
    """Untimed: repeat the step for about SETTLE_S seconds before the warm-up steps.  An idle MI355X needs some
    20-30 ms of sustained load to leave its low-power clocks (the first kernels of a process run ~25 % longer than
    the same kernels a few dozen launches later); a 5-step warm-up of sub-millisecond steps ends inside that ramp."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < SETTLE_S:
        for _ in range(10):
            step()
        sync()


def timed_steps(step, sync, steps, warmup):
    """The measurement protocol of every workload: (cold) `warmup` steps then `steps` timed steps straight after
    start-up, as a caller who does nothing special sees them; then the same again after settle().  Returns
    (ms per step settled, ms per step cold)."""
    out = []
    for settled in (False, True):
        if settled:
            settle(step, sync)
        for _ in range(warmup):
            step()
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        sync()
        out.append((time.perf_counter() - t0) * 1e3 / steps)
    return out[1], out[0]


def probe_cpu_opencl():
    """Looks for a CPU OpenCL device (PoCL or any other) through the ICD loader, the way the reference binds
    OpenCL (find_library('OpenCL'), clGetPlatformIDs, clGetDeviceIDs; minicl/api/OpenCL/OpenCL.py:16-23, 214-310).
    Runs in a child process so that a misbehaving ICD cannot disturb the measurement.  Returns a sentence."""
    import subprocess
    code = r"""
import ctypes, ctypes.util
name = ctypes.util.find_library('OpenCL')
if not name:
    print('no OpenCL ICD loader on this host'); raise SystemExit
cl = ctypes.CDLL(name)
n = ctypes.c_uint(0)
if cl.clGetPlatformIDs(0, None, ctypes.byref(n)) != 0 or n.value == 0:
    print('no CPU OpenCL device on this host (the ICD loader lists no platform)'); raise SystemExit
plats = (ctypes.c_void_p * n.value)()
cl.clGetPlatformIDs(n.value, plats, None)
found = []
for p in plats:
    buf = ctypes.create_string_buffer(256)
    cl.clGetPlatformInfo(ctypes.c_void_p(p), 0x0902, 256, buf, None)
    m = ctypes.c_uint(0)
    rc = cl.clGetDeviceIDs(ctypes.c_void_p(p), ctypes.c_ulong(2), 0, None, ctypes.byref(m))   # CL_DEVICE_TYPE_CPU
    if rc == 0 and m.value > 0:
        found.append(buf.value.decode())
print('CPU OpenCL device present on platform(s): ' + ', '.join(found) if found else
      'no CPU OpenCL device on this host (%d platform(s) listed by the ICD loader, none with a CPU device)' % n.value)
"""
    try:
        r = subprocess.run([sys.executable, '-c', code], capture_output=True, text=True, timeout=60)
        lines = [l for l in r.stdout.strip().splitlines() if l.strip()]
        return lines[-1] if lines else f'no CPU OpenCL device on this host (probe ended with status {r.returncode})'
    except Exception as e:   # noqa: BLE001
        return f'no CPU OpenCL device on this host (probe failed: {type(e).__name__})'


def bench_conv(api, name, steps, warmup, cpu=True, cpu_steps=3):
    xs, ws, s, d, padding, seed = CONV_CONFIGS[name]
    x, w, dy, ci = conv_tensors(xs, ws, s, d, padding, seed)
    N, C, IH, IW = xs
    O, _, KH, KW = ws
    desc = api.conv_desc(N, C, IH, IW, O, KH, KW, ci.OH, ci.OW, ci.PADL, ci.PADT, s, d)
    flops = 2.0 * N * O * ci.OH * ci.OW * C * KH * KW          # per pass
    nx, nw, ny = x.size, w.size, dy.size
    bytes_pass = {'fwd': 4.0 * (nx + nw + ny), 'dX': 4.0 * (ny + nw + 2 * nx), 'dW': 4.0 * (nx + ny + 2 * nw)}
    X, W, dY = Dev(api, x), Dev(api, w), Dev(api, dy)
    Y, dX, dW = Dev(api, shape=dy.shape), Dev(api, shape=xs), Dev(api, shape=ws)
    # As a training step runs it: the weights change once per step, so the copy in the kernels' layout that forward
    # and data gradient share (where the geometry's kernels read one) is made once per step, inside the forward pass.
    fwd_pw, dx_pw = api.conv2d_weights_plan(desc, api.PASS_FWD), api.conv2d_weights_plan(desc, api.PASS_DGRAD)
    in_place = KH * KW == 1                      # a 1x1 kernel already has the layout
    Wp = W if in_place or not (fwd_pw or dx_pw) else Dev(api, shape=(O, KH * KW, C))

    def p_fwd():
        if (fwd_pw or dx_pw) and not in_place:
            api.conv2d_permute_weights(0, desc, W.ptr, api.W_OIHW, Wp.ptr)
        if fwd_pw:
            api.conv2d_fwd_pw(0, desc, X.ptr, Wp.ptr, None, api.ACT_NONE, 0.0, Y.ptr, 0)
        else:
            api.conv2d_fwd(0, desc, X.ptr, W.ptr, Y.ptr, 0)

    def p_dx():
        if dx_pw:
            api.conv2d_dgrad_pw(0, desc, dY.ptr, Wp.ptr, dX.ptr, 1)
        else:
            api.conv2d_dgrad(0, desc, dY.ptr, W.ptr, dX.ptr, 1)

    passes = {'fwd': p_fwd, 'dX': p_dx, 'dW': lambda: api.conv2d_wgrad(0, desc, X.ptr, dY.ptr, dW.ptr, 1)}

    def step():
        for fn in passes.values():
            fn()

    wall_ms, cold_ms = timed_steps(step, lambda: api.synchronize(0), steps, warmup)

    per_pass = {}
    for k, fn in passes.items():
        ms = time_events(api, fn, max(steps, 5))
        per_pass[k] = {'ms': ms, 'tflops': flops / ms / 1e9, 'frac_mfma': flops / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS,
                       'alg_gbs': bytes_pass[k] / ms / 1e6, 'frac_hbm': bytes_pass[k] / ms / 1e6 / PEAK_HBM_GBS}
    dom = max(per_pass, key=lambda k: per_pass[k]['ms'])
    # the roofline that binds is the one whose minimum time is larger
    t_mfma = flops / (PEAK_FP32_MFMA_TFLOPS * 1e9)
    t_hbm = bytes_pass[dom] / (PEAK_HBM_GBS * 1e6)
    if t_mfma >= t_hbm:
        roof = {'bound': 'mfma', 'kernel': dom, 'achieved': per_pass[dom]['tflops'], 'peak': PEAK_FP32_MFMA_TFLOPS,
                'unit': 'TFLOP/s', 'frac': per_pass[dom]['frac_mfma'],
                'traffic': MEASURED_TRAFFIC_BYTES.get(name, {}).get(dom)}
    else:
        roof = {'bound': 'hbm', 'kernel': dom, 'achieved': per_pass[dom]['alg_gbs'], 'peak': PEAK_HBM_GBS,
                'unit': 'GB/s', 'frac': per_pass[dom]['frac_hbm'],
                'traffic': MEASURED_TRAFFIC_BYTES.get(name, {}).get(dom)}

    # parity on the very tensors that were timed (fresh outputs, no accumulation history)
    dX.zero()
    dW.zero()
    step()
    got = (Y.get(), dX.get(), dW.get())
    result = {
        'metric': 'conv2D fwd+bwd fp32 TFLOP/s', 'value': 3 * flops / wall_ms / 1e9, 'unit': 'TFLOP/s',
        'value_cold': 3 * flops / cold_ms / 1e9,
        'ms_per_step_cold': cold_ms, 'n_gpus': 1, 'steps': steps, 'warmup': warmup, 'settle_s': SETTLE_S, 'ms_per_step': wall_ms, 'higher_is_better': True,
        'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': f'{name}: x{list(xs)} w{list(ws)} stride {s} dilation {d} padding {padding!r}, '
                               'step = fwd + dX(+=) + dW(+=)'},
        'images_per_s': N / wall_ms * 1e3,
        'frac_mfma_peak_step': 3 * flops / wall_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS,
        'roofline': roof, 'passes': per_pass,
    }
    if flops < 1e9:   # a problem this small is a launch: say what a launch costs here
        floor = launch_floor_ms(api)
        result['launch_floor_ms'] = floor
        for k in per_pass:
            per_pass[k]['ms_min'] = min(time_events(api, passes[k], 300) for _ in range(3))
            per_pass[k]['x_launch_floor'] = per_pass[k]['ms_min'] / floor
    if cpu:
        from oracle import refpath
        cores = refpath.num_threads()
        ref = None
        times = []
        for i in range(cpu_steps + 1):
            t0 = time.perf_counter()
            ry = refpath.conv2d_fwd(x, w, s, d, padding)
            rdx = refpath.conv2d_dx(dy, w, xs, s, d, padding)
            rdw = refpath.conv2d_dw(x, dy, ws, s, d, padding)
            if i > 0:
                times.append(time.perf_counter() - t0)
            ref = (ry, rdx, rdw)
        cpu_s = float(np.median(times))
        result['cpu_baseline'] = {
            'value': 3 * flops / cpu_s / 1e12, 'unit': 'TFLOP/s', 'cores': cores, 'kind': 'port',
            'ms_per_step': cpu_s * 1e3,
            'sample': f'the full {name} step (fwd + dX + dW), median of {cpu_steps} after 1 warm-up, '
                      'C restatement of unfold -> register-tiled GeMM -> transpose incl. zero fills, OpenMP',
            'cpu_opencl': CPU_OPENCL}
        result['parity'] = {'checked_against': 'cpu_baseline outputs (fp32 reference data flow)',
                            'max_rel_err': max(rel_err(g, r) for g, r in zip(got, ref)), 'tolerance': 1e-4}
    for a in (X, W, dY, Y, dX, dW) + (() if Wp is W else (Wp,)):
        a.free()
    return result


def bench_matmul(api, steps, warmup, n=4096, cpu=True):
    rs = np.random.RandomState(0)
    a, b, dc = (rs.normal(0, 1, (n, n)).astype(np.float32) for _ in range(3))
    A, B, dC = Dev(api, a), Dev(api, b), Dev(api, dc)
    C, dA, dB = Dev(api, shape=(n, n)), Dev(api, shape=(n, n)), Dev(api, shape=(n, n))
    flops = 2.0 * n * n * n
    passes = {
        'fwd': lambda: api.gemm(0, 0, 0, 1, n, n, n, A.ptr, n, 0, B.ptr, n, 0, C.ptr, n, 0, 0),
        'dA': lambda: api.gemm(0, 0, 1, 1, n, n, n, dC.ptr, n, 0, B.ptr, n, 0, dA.ptr, n, 0, 1),
        'dB': lambda: api.gemm(0, 1, 0, 1, n, n, n, A.ptr, n, 0, dC.ptr, n, 0, dB.ptr, n, 0, 1),
    }

    def step():
        for fn in passes.values():
            fn()

    wall_ms, cold_ms = timed_steps(step, lambda: api.synchronize(0), steps, warmup)
    per_pass = {}
    for k, fn in passes.items():
        ms = time_events(api, fn, max(steps, 5))
        per_pass[k] = {'ms': ms, 'tflops': flops / ms / 1e9, 'frac_mfma': flops / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS}
    dom = max(per_pass, key=lambda k: per_pass[k]['ms'])
    dA.zero()
    dB.zero()
    step()
    res = {'metric': 'matmul fwd+dA+dB fp32 TFLOP/s', 'value': 3 * flops / wall_ms / 1e9, 'unit': 'TFLOP/s',
           'ms_per_step_cold': cold_ms, 'n_gpus': 1, 'steps': steps, 'warmup': warmup, 'settle_s': SETTLE_S, 'ms_per_step': wall_ms, 'higher_is_better': True,
           'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
           'config': {'workload': f'cfg2_matmul: [{n}x{n}] @ [{n}x{n}], step = C + dA(+=) + dB(+=)'},
           'roofline': {'bound': 'mfma', 'kernel': dom, 'achieved': per_pass[dom]['tflops'],
                        'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s', 'frac': per_pass[dom]['frac_mfma'],
                        'traffic': MEASURED_TRAFFIC_BYTES.get('cfg2_matmul', {}).get(dom) if n == 4096 else None},
           'passes': per_pass}
    if cpu:
        from oracle import refpath
        m = 1024   # bounded sample: the reference GeMM at 1024^3 (1/64 of the flops)
        t0 = time.perf_counter()
        refpath.matmul(a[:m, :m].copy(), b[:m, :m].copy())
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': 2.0 * m ** 3 / dt / 1e12, 'unit': 'TFLOP/s', 'cores': refpath.num_threads(),
                               'kind': 'port', 'sample': f'forward GeMM only at {m}^3, one run'}
        # parity of the full-size result on a row sample against fp64
        rows = np.arange(0, n, 257)
        c = C.get()
        res['parity'] = {'checked_against': 'fp64 numpy on every 257th row of C',
                         'max_rel_err': rel_err(c[rows], a[rows].astype(np.float64) @ b.astype(np.float64)),
                         'tolerance': 1e-4}
    for t in (A, B, dC, C, dA, dB):
        t.free()
    return res


def bench_dense(api, steps, warmup, batch=32, n_in=4096, n_out=4096, cpu=True):
    """Dense layer x[batch, in] @ w[in, out] + bias and its backward (module/Dense.py:44-48, matmul.py:64-72): at small
    batch every pass streams the weight matrix (or its gradient) once, so HBM and the matrix cores bound it about
    equally; each pass is reported against the larger of its two minimum times."""
    rs = np.random.RandomState(0)
    x = rs.uniform(-1, 1, (batch, n_in)).astype(np.float32)
    w = rs.normal(0, np.sqrt(2.0 / n_in), (n_in, n_out)).astype(np.float32)
    b = rs.normal(0, 0.1, n_out).astype(np.float32)
    dy = rs.normal(0, 1, (batch, n_out)).astype(np.float32)
    X, W, Bi, dY = Dev(api, x), Dev(api, w), Dev(api, b), Dev(api, dy)
    Y, dX, dW, dB = Dev(api, shape=(batch, n_out)), Dev(api, shape=(batch, n_in)), Dev(api, shape=(n_in, n_out)), Dev(api, shape=(n_out,))
    flops = 2.0 * batch * n_in * n_out
    nx, nw, ny = x.size, w.size, dy.size
    bytes_pass = {'fwd': 4.0 * (nx + nw + n_out + ny), 'dX': 4.0 * (ny + nw + 2 * nx), 'dW': 4.0 * (nx + ny + 2 * nw),
                  'dBias': 4.0 * (ny + 2 * n_out)}
    flops_pass = {'fwd': flops, 'dX': flops, 'dW': flops, 'dBias': 0.0}
    passes = {
        'fwd': lambda: api.gemm_bias_act(0, 0, 0, 1, batch, n_out, n_in, X.ptr, n_in, 0, W.ptr, n_out, 0, Bi.ptr,
                                         api.ACT_NONE, 0.0, Y.ptr, n_out, 0),
        'dX': lambda: api.gemm(0, 0, 1, 1, batch, n_in, n_out, dY.ptr, n_out, 0, W.ptr, n_out, 0, dX.ptr, n_in, 0, 1),
        'dW': lambda: api.gemm(0, 1, 0, 1, n_in, n_out, batch, X.ptr, n_in, 0, dY.ptr, n_out, 0, dW.ptr, n_out, 0, 1),
        'dBias': lambda: api.bias_act_bwd(0, batch, n_out, 1, None, dY.ptr, api.ACT_NONE, 0.0, None, dB.ptr, 1),
    }

    def step():
        for fn in passes.values():
            fn()

    wall_ms, cold_ms = timed_steps(step, lambda: api.synchronize(0), steps, warmup)
    per_pass = {}
    for k, fn in passes.items():
        ms = time_events(api, fn, max(steps, 20))
        t_mfma = flops_pass[k] / (PEAK_FP32_MFMA_TFLOPS * 1e9)    # ms
        t_hbm = bytes_pass[k] / (PEAK_HBM_GBS * 1e6)
        per_pass[k] = {'ms': ms, 'tflops': flops_pass[k] / ms / 1e9, 'frac_mfma': t_mfma / ms,
                       'alg_gbs': bytes_pass[k] / ms / 1e6, 'frac_hbm': t_hbm / ms,
                       'bound': 'mfma' if t_mfma >= t_hbm else 'hbm', 'frac_roofline': max(t_mfma, t_hbm) / ms}
    # the dominant kernel: the pass furthest below its roofline among the three products
    dom = min(('fwd', 'dX', 'dW'), key=lambda k: per_pass[k]['frac_roofline'])
    pp = per_pass[dom]
    if pp['bound'] == 'mfma':
        roof = {'bound': 'mfma', 'kernel': dom, 'achieved': pp['tflops'], 'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                'frac': pp['frac_mfma']}
    else:
        roof = {'bound': 'hbm', 'kernel': dom, 'achieved': pp['alg_gbs'], 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                'frac': pp['frac_hbm']}
    name = f'cfgM_dense_b{batch}'
    roof['traffic'] = MEASURED_TRAFFIC_BYTES.get(name, {}).get(dom)
    dX.zero()
    dW.zero()
    dB.zero()
    step()
    res = {'metric': 'dense layer fwd+bwd fp32 TFLOP/s', 'value': 3 * flops / wall_ms / 1e9, 'unit': 'TFLOP/s',
           'ms_per_step_cold': cold_ms, 'n_gpus': 1, 'steps': steps, 'warmup': warmup, 'settle_s': SETTLE_S,
           'ms_per_step': wall_ms, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32',
           'data': 'synthetic',
           'config': {'workload': f'{name}: x[{batch}, {n_in}] @ w[{n_in}, {n_out}] + bias, '
                                  'step = fwd(+bias) + dX(+=) + dW(+=) + dBias(+=)'},
           'samples_per_s': batch / wall_ms * 1e3, 'roofline': roof, 'passes': per_pass}
    if cpu:
        from oracle import refpath
        times = []
        ref = None
        for i in range(3):
            t0 = time.perf_counter()
            ry = refpath.matmul(x, w) + b
            rdx, rdw = refpath.matmul_bwd(x, w, dy)
            if i > 0:
                times.append(time.perf_counter() - t0)
            ref = (ry, rdx, rdw)
        cpu_s = float(np.median(times))
        res['cpu_baseline'] = {'value': 3 * flops / cpu_s / 1e12, 'unit': 'TFLOP/s', 'cores': refpath.num_threads(),
                               'kind': 'port', 'ms_per_step': cpu_s * 1e3,
                               'sample': 'the full step (register-tiled GeMM forward, materialised transposes + GeMM for '
                                         'both gradients, numpy bias add), median of 2 after 1 warm-up',
                               'cpu_opencl': CPU_OPENCL}
        got = (Y.get(), dX.get(), dW.get())
        res['parity'] = {'checked_against': 'cpu_baseline outputs (fp32 reference data flow)',
                         'max_rel_err': max(rel_err(g, r) for g, r in zip(got, ref)),
                         'dbias_rel_err': rel_err(dB.get(), dy.astype(np.float64).sum(0)), 'tolerance': 1e-4}
    for t in (X, W, Bi, dY, Y, dX, dW, dB):
        t.free()
    return res


def bench_conv_transpose(api, steps, warmup, cpu=True):
    """Decoder layer: conv2DTranspose 256 -> 128, 5x5, stride 2, 'same', 16x16 -> 32x32, batch 16.  The three
    passes run on the convolution kernels with the roles swapped (forward = dgrad, dI = forward, dK = wgrad)."""
    N, IC, IH, IW, OC, KS, S = 16, 256, 16, 16, 128, 5, 2
    ci = conv_info((N, IC, IH, IW), (OC, IC, KS, KS), S, 1, 'same')
    rs = np.random.RandomState(0)
    x = rs.uniform(-1, 1, (N, IC, IH, IW)).astype(np.float32)
    k = rs.normal(0, np.sqrt(2.0 / (IC * KS * KS)), (OC, IC, KS, KS)).astype(np.float32)
    dy = rs.normal(0, 1, (N, OC, ci.OH_T, ci.OW_T)).astype(np.float32)
    desc = api.conv_desc(N, OC, ci.OH_T, ci.OW_T, IC, KS, KS, IH, IW, ci.PADL, ci.PADT, S, 1)
    X, K, dY = Dev(api, x), Dev(api, k), Dev(api, dy)
    Y, dI, dK = Dev(api, shape=dy.shape), Dev(api, shape=x.shape), Dev(api, shape=k.shape)
    flops = 2.0 * N * IC * IH * IW * OC * KS * KS

    # The kernel is stored (OC, IC, KH, KW): relative to the borrowed convolution (OC channels in, IC out) its channel
    # axes are swapped.  The copy in the kernels' layout is made straight from that storage, once per step (the
    # weights change once per step), and the kernel gradient is written straight into that storage.
    Wp = Dev(api, shape=(IC, KS * KS, OC))

    def p_wp():
        api.conv2d_permute_weights(0, desc, K.ptr, api.W_IOHW, Wp.ptr)

    def p_fwd():
        api.conv2d_dgrad_pw(0, desc, X.ptr, Wp.ptr, Y.ptr, 0)

    def p_di():
        api.conv2d_fwd_pw(0, desc, dY.ptr, Wp.ptr, None, api.ACT_NONE, 0.0, dI.ptr, 1)

    def p_dk():
        api.conv2d_wgrad_iohw(0, desc, dY.ptr, X.ptr, dK.ptr, 1)

    passes = {'weights': p_wp, 'fwd': p_fwd, 'dI': p_di, 'dK': p_dk}

    def step():
        for fn in passes.values():
            fn()

    wall_ms, cold_ms = timed_steps(step, lambda: api.synchronize(0), steps, warmup)
    per_pass = {}
    for name, fn in passes.items():
        ms = time_events(api, fn, max(steps, 5))
        if name == 'weights':   # the copy of the kernel in the kernels' layout: bytes, no arithmetic
            per_pass[name] = {'ms': ms, 'alg_gbs': 2 * 4.0 * k.size / ms / 1e6, 'frac_hbm': 2 * 4.0 * k.size / ms / 1e6 / PEAK_HBM_GBS,
                              'note': 'one launch per step here; in a training step through the Python API the optimizer '
                                      'update writes this copy and the launch does not exist'}
        else:
            per_pass[name] = {'ms': ms, 'tflops': flops / ms / 1e9, 'frac_mfma': flops / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS}
    dom = max(('fwd', 'dI', 'dK'), key=lambda n: per_pass[n]['ms'])
    dI.zero()
    dK.zero()
    step()
    res = {'metric': 'conv2DTranspose fwd+bwd fp32 TFLOP/s', 'value': 3 * flops / wall_ms / 1e9, 'unit': 'TFLOP/s',
           'ms_per_step_cold': cold_ms, 'n_gpus': 1, 'steps': steps, 'warmup': warmup, 'settle_s': SETTLE_S, 'ms_per_step': wall_ms, 'higher_is_better': True,
           'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
           'config': {'workload': f'cfgT_decoder: conv2DTranspose x[{N}, {IC}, {IH}, {IW}] k[{OC}, {IC}, {KS}, {KS}] '
                                  f"stride {S} 'same', step = weight copy + fwd + dI(+=) + dK(+=)"},
           'roofline': {'bound': 'mfma', 'kernel': dom, 'achieved': per_pass[dom]['tflops'],
                        'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s', 'frac': per_pass[dom]['frac_mfma'],
                        'traffic': MEASURED_TRAFFIC_BYTES.get('cfgT_decoder', {}).get(dom)},
           'passes': per_pass}
    if cpu:
        from oracle import conv2d_transpose_all
        t0 = time.perf_counter()
        ry, rdi, rdk = conv2d_transpose_all(x[:2], k, dy[:2], S, 1, 'same')
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': 3 * flops * 2 / N / dt / 1e12, 'unit': 'TFLOP/s', 'cores': 1, 'kind': 'port',
                               'sample': 'numpy fp64 oracle (unfold + matmul), 2 of the 16 images, one run'}
        got_y, got_di = Y.get()[:2], dI.get()[:2]
        res['parity'] = {'checked_against': 'fp64 oracle on images 0-1 (Y, dI)',
                         'max_rel_err': max(rel_err(got_y, ry), rel_err(got_di, rdi)), 'tolerance': 1e-4}
    for t in (X, K, dY, Wp, Y, dI, dK):
        t.free()
    return res


def bench_depthwise(api, steps, warmup, cpu=True):
    """Depthwise 3x3 'same' on x[32, 256, 56, 56]: no contraction over channels, so the roofline that binds is
    HBM: forward reads X and writes Y (K is 9 KB), dX reads dY and reads + writes dX, dK reads X and dY."""
    N, C, H, KS = 32, 256, 56, 3
    ci = conv_info((N, C, H, H), (C, C, KS, KS), 1, 1, 'same')
    rs = np.random.RandomState(0)
    x = rs.uniform(-1, 1, (N, C, H, H)).astype(np.float32)
    k = rs.normal(0, 0.5, (C, KS, KS)).astype(np.float32)
    dy = rs.normal(0, 1, (N, C, ci.OH, ci.OW)).astype(np.float32)
    desc = api.conv_desc(N, C, H, H, C, KS, KS, ci.OH, ci.OW, ci.PADL, ci.PADT, 1, 1)
    X, K, dY = Dev(api, x), Dev(api, k), Dev(api, dy)
    Y, dX, dK = Dev(api, shape=dy.shape), Dev(api, shape=x.shape), Dev(api, shape=k.shape)
    nx, ny, nk = x.size, dy.size, k.size
    bytes_pass = {'fwd': 4.0 * (nx + ny + nk), 'dX': 4.0 * (ny + 2 * nx + nk), 'dK': 4.0 * (nx + ny + 2 * nk)}
    passes = {
        'fwd': lambda: api.depthwise_conv2d_fwd(0, desc, X.ptr, K.ptr, Y.ptr, 0),
        'dX': lambda: api.depthwise_conv2d_dgrad(0, desc, dY.ptr, K.ptr, dX.ptr, 1),
        'dK': lambda: api.depthwise_conv2d_wgrad(0, desc, X.ptr, dY.ptr, dK.ptr, 1),
    }

    def step():
        for fn in passes.values():
            fn()

    wall_ms, cold_ms = timed_steps(step, lambda: api.synchronize(0), steps, warmup)
    # Per pass INSIDE the step: launched back to back, a pass finds its 100-200 MB working set in the 256 MB memory-side
    # cache and looks faster than any caller will see it (the back-to-back figure is kept beside it for comparison).
    names = {'depthwise_conv2d_fwd': 'fwd', 'depthwise_conv2d_dgrad': 'dX', 'depthwise_conv2d_wgrad': 'dK'}
    with InStepTimer(api, list(names), lambda name, args: names[name]) as timer:
        for _ in range(3):
            step()
        api.synchronize(0)
        timer.per_step_ms(1)
        for _ in range(max(steps, 20)):
            step()
        api.synchronize(0)
        in_step = timer.per_step_ms(max(steps, 20))
    per_pass = {}
    for name, fn in passes.items():
        ms = in_step[name]
        per_pass[name] = {'ms': ms, 'alg_gbs': bytes_pass[name] / ms / 1e6,
                          'frac_hbm': bytes_pass[name] / ms / 1e6 / PEAK_HBM_GBS, 'frac_mfma': 0.0,
                          'ms_back_to_back': time_events(api, fn, max(steps, 5))}
    dom = min(per_pass, key=lambda n: per_pass[n]['frac_hbm'])
    dX.zero()
    dK.zero()
    step()
    total_bytes = sum(bytes_pass.values())
    res = {'metric': 'depthwise_conv2D fwd+bwd algorithmic GB/s', 'value': total_bytes / wall_ms / 1e6, 'unit': 'GB/s',
           'ms_per_step_cold': cold_ms, 'n_gpus': 1, 'steps': steps, 'warmup': warmup, 'settle_s': SETTLE_S, 'ms_per_step': wall_ms, 'higher_is_better': True,
           'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
           'config': {'workload': f"cfgD_depthwise: x[{N}, {C}, {H}, {H}] k[{C}, {KS}, {KS}] stride 1 'same', "
                                  'step = fwd + dX(+=) + dK(+=)'},
           'images_per_s': N / wall_ms * 1e3,
           'roofline': {'bound': 'hbm', 'kernel': dom, 'achieved': per_pass[dom]['alg_gbs'], 'peak': PEAK_HBM_GBS,
                        'unit': 'GB/s', 'frac': per_pass[dom]['frac_hbm'],
                        'traffic': MEASURED_TRAFFIC_BYTES.get('cfgD_depthwise', {}).get(dom)},
           'passes': per_pass}
    if cpu:
        from oracle import depthwise_all
        t0 = time.perf_counter()
        ry, rdx, rdk = depthwise_all(x[:4], k, dy[:4], 1, 1, 'same')
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': total_bytes * 4 / N / dt / 1e9, 'unit': 'GB/s', 'cores': 1, 'kind': 'port',
                               'sample': 'numpy fp64 oracle, 4 of the 32 images, one run'}
        res['parity'] = {'checked_against': 'fp64 oracle on images 0-3 (Y, dX)',
                         'max_rel_err': max(rel_err(Y.get()[:4], ry), rel_err(dX.get()[:4], rdx)), 'tolerance': 1e-4}
    for t in (X, K, dY, Y, dX, dK):
        t.free()
    return res


ENC_CHANS = [3, 64, 128, 256, 512]


def _encoder(nn, ws):
    layers = [nn.Conv2D(ENC_CHANS[i], ENC_CHANS[i + 1], 5, stride=2, padding=2, kernel_initializer=nn.initializer.NumpyArray(ws[i]))
              for i in range(4)]

    class Enc(nn.Module):
        def __init__(self):
            self.convs = layers

        def forward(self, x):
            for i, c in enumerate(self.convs):
                x = c(x)
                if i < 3:
                    x = nn.leaky_relu(x, 0.1)
            return x

    return Enc(), layers


def _encoder_conv_passes(nn, api, step, steps):
    """Every convolution pass of the encoder step timed inside the step (HIP events around the library call, on the
    library's stream).  Returns {'L<layer>_<pass>': (ms, flops)}."""
    layer_of = {c: i + 1 for i, c in enumerate(ENC_CHANS[:4])}
    kind = {'conv2d_fwd_pw': 'fwd', 'conv2d_fwd_bias_act': 'fwd', 'conv2d_fwd': 'fwd', 'conv2d_dgrad_pw': 'dX', 'conv2d_dgrad': 'dX',
            'conv2d_wgrad': 'dW'}

    def label(name, args):
        d = args[1]
        return f'L{layer_of[d.C]}_{kind[name]}', 2.0 * d.N * d.O * d.OH * d.OW * d.C * d.KH * d.KW

    with InStepTimer(api, list(kind), label) as timer:
        for _ in range(3):
            step()
        nn.devices.wait()
        timer.per_step_ms(1)
        for _ in range(steps):
            step()
        nn.devices.wait()
        ms = timer.per_step_ms(steps)
    return {name: (t, flops) for (name, flops), t in sorted(ms.items())}


def bench_encoder(steps, warmup, cpu=True):
    """cfg5: full training step (forward, backward, SGD) of the 4-layer 5x5
    stride-2 encoder through the litenn-compatible Python API."""
    import contextlib
    with contextlib.redirect_stdout(sys.stderr):   # the device banner must not share stdout with the JSON line
        import litenn_amd as nn
        nn.devices.get_current()
    from litenn_amd.core.hip import api
    N = 16
    rs = np.random.RandomState(0)
    x_n = rs.uniform(-1, 1, (N, 3, 128, 128)).astype(np.float32)
    ws = [rs.normal(0, np.sqrt(2.0 / (ENC_CHANS[i] * 25)), (ENC_CHANS[i + 1], ENC_CHANS[i], 5, 5)).astype(np.float32)
          for i in range(4)]
    enc, layers = _encoder(nn, ws)
    opt = nn.optimizer.SGD(enc.trainables(), lr=1e-3)
    x_t = nn.Tensor_from_value(x_n)

    last = {}

    def step():
        opt.zero_grad()
        loss = nn.square(enc(x_t)).mean()
        loss.backward()
        opt.step()
        last['loss'] = loss

    wall_ms, cold_ms = timed_steps(step, nn.devices.wait, steps, warmup)
    final_loss = float(last['loss'].np()[0])
    last.clear()
    # the convolution passes of the step, each timed inside the step (HIP events), and what is left for the helpers
    conv = _encoder_conv_passes(nn, api, step, max(steps, 20))
    last.clear()
    conv_ms = sum(ms for ms, _ in conv.values())
    conv_flops = sum(fl for _, fl in conv.values())
    dom = min((k for k in conv if not k.startswith('L1_')), key=lambda k: conv[k][1] / conv[k][0])   # lowest TFLOP/s
    dom_tflops = conv[dom][1] / conv[dom][0] / 1e9
    # helper launches: leaky_relu forward / backward on the three inner activations, square + mean and their backward
    # on the last, bias gradients (one pass over each dY), the SGD update (read W and G, write W, the accumulator and
    # the permuted copy of W): algorithmic bytes
    act = [N * ENC_CHANS[i + 1] * (128 >> (i + 1)) ** 2 for i in range(4)]
    n_w = sum(w.size for w in ws)
    helper_bytes = 4.0 * (sum(2 * a + 3 * a for a in act[:3]) + 2 * act[3] + act[3] + 3 * act[3] + sum(act) + 5 * n_w)
    helper_ms = max(wall_ms - conv_ms, 1e-6)
    res = {'metric': 'encoder training step images/s', 'value': N / wall_ms * 1e3, 'unit': 'images/s', 'n_gpus': 1,
           'steps': steps, 'warmup': warmup, 'settle_s': SETTLE_S, 'ms_per_step': wall_ms, 'ms_per_step_cold': cold_ms,
           'value_cold': N / cold_ms * 1e3, 'higher_is_better': True, 'scaling': 'weak',
           'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
           'config': {'workload': 'cfg5_encoder: 16x3x128x128, 3->64->128->256->512, 5x5 s2 p2, leaky_relu(0.1), '
                                  'loss mean(square), SGD lr 1e-3; forward + backward + update'},
           'conv_tflops': conv_flops / wall_ms / 1e9, 'frac_mfma_peak_step': conv_flops / wall_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS,
           'final_loss': final_loss,
           'roofline': {'bound': 'mfma', 'kernel': dom, 'achieved': dom_tflops, 'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                        'frac': dom_tflops / PEAK_FP32_MFMA_TFLOPS,
                        'traffic': MEASURED_TRAFFIC_BYTES.get('cfg5_encoder', {}).get(dom)},
           'conv_share': {'ms': conv_ms, 'tflops': conv_flops / conv_ms / 1e9,
                          'frac_mfma': conv_flops / conv_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS},
           'helper_share': {'ms': helper_ms, 'alg_bytes': helper_bytes, 'alg_gbs': helper_bytes / helper_ms / 1e6,
                            'frac_hbm': helper_bytes / helper_ms / 1e6 / PEAK_HBM_GBS,
                            'note': 'step time not spent in the convolution passes (timed inside the step): pointwise, bias '
                                    'gradient, loss and optimizer launches, and the gaps between launches'},
           'passes': {k: {'ms': ms, 'tflops': fl / ms / 1e9, 'frac_mfma': fl / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS}
                      for k, (ms, fl) in conv.items()}}
    del x_t, opt, enc, layers
    if cpu:
        from oracle import refpath, conv2d_fwd, conv2d_dx, conv2d_dw
        # CPU baseline: the reference data flow of every convolution pass of the step (unfold -> GeMM -> transpose,
        # zero fills included), composed per layer on the batch of 16, one run; pointwise work is not included
        t0 = time.perf_counter()
        a = x_n
        acts = [a]
        for i in range(4):
            a = refpath.conv2d_fwd(a, ws[i], 2, 1, 2)
            acts.append(a)
        g = acts[4]
        for i in (3, 2, 1, 0):
            refpath.conv2d_dw(acts[i], g, ws[i].shape, 2, 1, 2)
            if i > 0:
                g = refpath.conv2d_dx(g, ws[i], acts[i].shape, 2, 1, 2)
        cpu_s = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': N / cpu_s, 'unit': 'images/s', 'cores': refpath.num_threads(), 'kind': 'port',
                               'ms_per_step': cpu_s * 1e3, 'conv_tflops': conv_flops / cpu_s / 1e12,
                               'sample': 'the 11 convolution passes of one step at batch 16 (C restatement of unfold -> '
                                         'register-tiled GeMM -> transpose incl. zero fills, OpenMP), one run; pointwise, '
                                         'loss and optimizer work not included',
                               'cpu_opencl': CPU_OPENCL}
        # parity: one training step on 2 images against the fp64 restatement (loss, first and last updated kernel)
        enc2, layers2 = _encoder(nn, ws)
        opt2 = nn.optimizer.SGD(enc2.trainables(), lr=1e-3)
        x2 = x_n[:2]
        x2_t = nn.Tensor_from_value(x2)
        loss2 = nn.square(enc2(x2_t)).mean()
        loss2.backward()
        got_dw = {i: layers2[i].kernel.get_grad().np().astype(np.float64) for i in (0, 3)}
        opt2.step()
        W = [w.astype(np.float64) for w in ws]
        acts, zs = [x2.astype(np.float64)], []
        for i in range(4):
            z = conv2d_fwd(acts[-1], W[i], 2, 1, 2)
            zs.append(z)
            acts.append(np.where(z >= 0, z, 0.1 * z) if i < 3 else z)
        ref_loss = (zs[3] ** 2).mean()
        dz = 2 * zs[3] / zs[3].size
        errs = {}
        for i in (3, 2, 1, 0):
            dw = conv2d_dw(acts[i], dz, W[i].shape, 2, 1, 2)
            if i in got_dw:
                errs[f'dW{i + 1}'] = rel_err(got_dw[i], dw)
                errs[f'W{i + 1}_updated'] = rel_err(layers2[i].kernel.np(), W[i] - 1e-3 * dw)
            if i > 0:
                dz = conv2d_dx(dz, W[i], acts[i].shape, 2, 1, 2) * np.where(zs[i - 1] >= 0, 1.0, 0.1)
        res['parity'] = {'checked_against': 'fp64 restatement of one training step on 2 images',
                         'loss_rel_err': abs(float(loss2.np()[0]) - ref_loss) / abs(ref_loss),
                         'max_rel_err': max(errs.values()), 'what': 'kernel gradients and updated kernels of layers 1 and 4',
                         'each': errs, 'tolerance': 1e-4}
        del x2_t, opt2, enc2, layers2, loss2
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--all', action='store_true', help='also measure every benchmark configuration')
    ap.add_argument('--out-dir', default='.', help='where --all writes bench_all.jsonl')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='run only a plain device copy of 256 MiB (three launches of the element-wise kernel) and exit: '
                         'the reference reading for the FETCH_SIZE / WRITE_SIZE counters')
    ap.add_argument('--config', default='cfg3_vgg3x3', choices=list(CONV_CONFIGS) + ['cfg2_matmul', 'cfg5_encoder', 'cfgT_decoder', 'cfgD_depthwise', 'cfgM_dense', 'cfgM_dense_b32', 'cfgM_dense_b256'],
                    help='workload of the JSON line (default: the headline configuration)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)')
    global CPU_OPENCL
    if not args.no_cpu:
        CPU_OPENCL = probe_cpu_opencl()          # before this process touches the GPU
    from litenn_amd.core.hip import api
    if api.device_count() < 1:
        sys.exit('bench.py needs an MI355X: no HIP device is visible')
    if args.copy_calibration:
        n = 1 << 26
        src, dst = Dev(api, shape=(n,)), Dev(api, shape=(n,))
        src.zero()
        for _ in range(3):
            api.ew_fwd(0, api.EW_ADD_CONST, n, src.ptr, dst.ptr, 0.0, 0)
        api.synchronize(0)
        print(json.dumps({'copy_calibration': {'kernel': 'ew_fwd_kernel', 'launches': 3, 'read_bytes': 4 * n,
                                               'write_bytes': 4 * n}}), flush=True)
        return
    if args.all:
        os.makedirs(args.out_dir, exist_ok=True)
        with open(os.path.join(args.out_dir, 'bench_all.jsonl'), 'w') as f:
            for name in CONV_CONFIGS:
                if name == 'cfg3_vgg3x3':
                    continue
                r = bench_conv(api, name, args.steps, args.warmup, cpu=not args.no_cpu, cpu_steps=1)
                f.write(json.dumps(r) + '\n')
                f.flush()
                print(f'[bench] {name}: {r["value"]:.1f} TFLOP/s step, passes '
                      + ', '.join(f'{k} {v["ms"]:.3f} ms' for k, v in r['passes'].items()), file=sys.stderr, flush=True)
            r = bench_matmul(api, args.steps, args.warmup, cpu=not args.no_cpu)
            f.write(json.dumps(r) + '\n')
            print(f'[bench] cfg2 matmul: {r["value"]:.1f} TFLOP/s', file=sys.stderr, flush=True)
            r = bench_conv_transpose(api, args.steps, args.warmup, cpu=not args.no_cpu)
            f.write(json.dumps(r) + '\n')
            print(f'[bench] cfgT decoder: {r["value"]:.1f} TFLOP/s', file=sys.stderr, flush=True)
            r = bench_depthwise(api, args.steps, args.warmup, cpu=not args.no_cpu)
            f.write(json.dumps(r) + '\n')
            print(f'[bench] cfgD depthwise: {r["value"]:.0f} GB/s', file=sys.stderr, flush=True)
            for bsz in (32, 256):
                r = bench_dense(api, args.steps, args.warmup, batch=bsz, cpu=not args.no_cpu)
                f.write(json.dumps(r) + '\n')
                print(f'[bench] cfgM dense batch {bsz}: ' + ', '.join(f'{k} {v["ms"] * 1e3:.1f} us' for k, v in r['passes'].items()),
                      file=sys.stderr, flush=True)
            r = bench_encoder(args.steps, args.warmup, cpu=not args.no_cpu)
            f.write(json.dumps(r) + '\n')
            print(f'[bench] cfg5 encoder: {r["value"]:.0f} images/s, {r["ms_per_step"]:.3f} ms/step', file=sys.stderr,
                  flush=True)
    if args.config in ('cfgM_dense', 'cfgM_dense_b32'):
        res = bench_dense(api, args.steps, args.warmup, batch=32, cpu=not args.no_cpu)
        if args.config == 'cfgM_dense':   # the same layer at a batch where the matrix cores bound every pass
            res['batch256'] = bench_dense(api, args.steps, args.warmup, batch=256, cpu=not args.no_cpu)
    elif args.config == 'cfgM_dense_b256':
        res = bench_dense(api, args.steps, args.warmup, batch=256, cpu=not args.no_cpu)
    elif args.config == 'cfg2_matmul':
        res = bench_matmul(api, args.steps, args.warmup, cpu=not args.no_cpu)
    elif args.config == 'cfg5_encoder':
        res = bench_encoder(args.steps, args.warmup, cpu=not args.no_cpu)
    elif args.config == 'cfgT_decoder':
        res = bench_conv_transpose(api, args.steps, args.warmup, cpu=not args.no_cpu)
    elif args.config == 'cfgD_depthwise':
        res = bench_depthwise(api, args.steps, args.warmup, cpu=not args.no_cpu)
    else:
        res = bench_conv(api, args.config, args.steps, args.warmup, cpu=not args.no_cpu)
    if args.all:
        with open(os.path.join(args.out_dir, 'bench_all.jsonl'), 'a') as f:
            f.write(json.dumps(res) + '\n')
    print(json.dumps(res), flush=True)


if __name__ == '__main__':
    main()
