"""The litenn-compatible Python layer: the reference's own self-tests restated
(conv2d_test conv2D.py:76-126, matmul_test matmul.py:167-234, transpose_test
transpose.py:106-163, backward_test test.py:166-195, Conv2D_test / Dense_test,
shallow_mode_test test.py:147-164, SGD_test test.py:265-270) plus behaviour the
user guide documents.  Every test runs twice: on the numpy stand-in (host
logic, no GPU) and - marked gpu - on the real library."""
import itertools

import numpy as np
import pytest

from oracle import conv2d_all, conv2d_transpose_all, depthwise_all, hash_rng, info_conv2d


def test_conv2d_reference_style(nn_backend):
    nn = nn_backend
    rs = np.random.RandomState(0)
    n_cases = 0
    for padding, dilation, stride, ks in itertools.product(['same', 'valid', 0, 2], [1, 2], [1, 2, 3], [5, 3, 1]):
        for n, ic, oc, hw in [(1, 1, 1, 8), (4, 2, 4, 8), (1, 4, 2, 16)]:
            if padding == 'valid' and hw < ks:
                continue
            input_n = rs.randint(2 ** 4, size=(n, ic, hw, hw)).astype(np.float32)
            kernel_n = rs.randint(2 ** 4, size=(oc, ic, ks, ks)).astype(np.float32)
            input_t = nn.Tensor_from_value(input_n)
            kernel_t = nn.Tensor_from_value(kernel_n)
            conved_t = nn.conv2D(input_t, kernel_t, stride=stride, dilation=dilation, padding=padding)
            grad_n = rs.randint(2 ** 4, size=tuple(conved_t.shape)).astype(np.float32)
            y, dI, dK = conv2d_all(input_n, kernel_n, grad_n, stride, dilation, padding)
            assert y.shape == conved_t.shape
            assert np.array_equal(conved_t.np(), y)
            input_t.get_grad().fill(1.0)
            kernel_t.get_grad().fill(1.0)
            nn.backward({conved_t: grad_n}, grad_for_non_trainables=True)
            assert np.array_equal(input_t.get_grad().np() - 1.0, dI)
            assert np.array_equal(kernel_t.get_grad().np() - 1.0, dK)
            n_cases += 1
    assert n_cases > 150


def test_conv2d_transpose_reference_style(nn_backend):
    """conv2DTranspose_test (conv2DTranspose.py:74-126): its whole grid, exact
    on integer-valued data, gradients accumulated onto a pre-filled 1.0; a
    dilation-2 column is added."""
    nn = nn_backend
    rs = np.random.RandomState(1)
    n_cases = 0
    for padding, dilation, stride, ks, n, ic, oc, hw in itertools.product(
            ['same', 'valid'], [1, 2], [3, 2, 1], [1, 3, 5, 7], [4, 1], [1, 4], [1, 4], [16, 8, 4]):
        if padding == 'valid' and hw < ks:
            continue
        if dilation == 2 and (n, hw) != (1, 8):
            continue
        input_n = rs.randint(2 ** 4, size=(n, ic, hw, hw)).astype(np.float32)
        kernel_n = rs.randint(2 ** 4, size=(oc, ic, ks, ks)).astype(np.float32)
        input_t = nn.Tensor_from_value(input_n)
        kernel_t = nn.Tensor_from_value(kernel_n)
        conved_t = nn.conv2DTranspose(input_t, kernel_t, stride=stride, dilation=dilation, padding=padding)
        grad_n = rs.randint(2 ** 4, size=tuple(conved_t.shape)).astype(np.float32)
        y, dI, dK = conv2d_transpose_all(input_n, kernel_n, grad_n, stride, dilation, padding)
        assert y.shape == conved_t.shape
        assert np.array_equal(conved_t.np(), y), (padding, dilation, stride, ks, n, ic, oc, hw)
        input_t.get_grad().fill(1.0)
        kernel_t.get_grad().fill(1.0)
        nn.backward({conved_t: grad_n}, grad_for_non_trainables=True)
        assert np.array_equal(input_t.get_grad().np() - 1.0, dI), (padding, dilation, stride, ks, n, ic, oc, hw)
        assert np.array_equal(kernel_t.get_grad().np() - 1.0, dK), (padding, dilation, stride, ks, n, ic, oc, hw)
        n_cases += 1
    assert n_cases > 250


def test_conv2d_transpose_wide_channels(nn_backend):
    """Channel counts for which the borrowed convolution passes read the kernel in their own permuted layout: the
    copy is made straight from the kernel as stored, and the kernel gradient is written straight into its layout."""
    nn = nn_backend
    rs = np.random.RandomState(4)
    for n, ic, oc, hw, ks, stride, padding in [(2, 32, 8, 6, 3, 2, 'same'), (1, 32, 32, 5, 5, 2, 'same'),
                                                (2, 64, 32, 4, 3, 1, 'valid'), (1, 32, 36, 7, 4, 2, 'valid'),
                                                (2, 96, 64, 3, 1, 1, 'same')]:
        input_n = rs.randint(-3, 4, size=(n, ic, hw, hw)).astype(np.float32)
        kernel_n = rs.randint(-3, 4, size=(oc, ic, ks, ks)).astype(np.float32)
        input_t, kernel_t = nn.Tensor_from_value(input_n), nn.Tensor_from_value(kernel_n)
        out_t = nn.conv2DTranspose(input_t, kernel_t, stride=stride, padding=padding)
        grad_n = rs.randint(-3, 4, size=tuple(out_t.shape)).astype(np.float32)
        y, dI, dK = conv2d_transpose_all(input_n, kernel_n, grad_n, stride, 1, padding)
        assert np.array_equal(out_t.np(), y), (n, ic, oc, hw, ks, stride, padding)
        input_t.get_grad().fill(1.0)
        kernel_t.get_grad().fill(1.0)
        nn.backward({out_t: grad_n}, grad_for_non_trainables=True)
        assert np.array_equal(input_t.get_grad().np() - 1.0, dI), (n, ic, oc, hw, ks, stride, padding)
        assert np.array_equal(kernel_t.get_grad().np() - 1.0, dK), (n, ic, oc, hw, ks, stride, padding)


def test_permuted_weight_copy_is_shared_and_follows_the_weights(nn_backend, monkeypatch):
    """Forward and data gradient read one cached copy of the kernel in the kernels' layout; an optimizer step writes
    the new values into the copy as well, and the copy is made again only after the kernel's contents may have changed
    otherwise (set, fill); results stay exact."""
    nn = nn_backend
    from litenn_amd.core.hip import api
    made = []
    real = api.conv2d_permute_weights
    monkeypatch.setattr(api, 'conv2d_permute_weights', lambda *a: (made.append(1), real(*a))[1])
    rs = np.random.RandomState(9)
    x_n = rs.randint(-2, 3, size=(2, 32, 7, 7)).astype(np.float32)
    k_n = rs.randint(-2, 3, size=(32, 32, 3, 3)).astype(np.float32)
    x_t, k_t = nn.Tensor_from_value(x_n), nn.Tensor_from_value(k_n)
    opt = nn.optimizer.SGD([k_t], lr=0.5)

    def step(expect_k):
        y = nn.conv2D(x_t, k_t, stride=2)
        g_n = np.ones(tuple(y.shape), np.float32)
        ry, rdx, rdw = conv2d_all(x_n, expect_k, g_n, 2, 1, 'same')
        assert np.array_equal(y.np(), ry)
        opt.zero_grad()
        nn.backward({y: g_n}, grad_for_non_trainables=True)
        assert np.array_equal(x_t.get_grad().np(), rdx) and np.array_equal(k_t.get_grad().np(), rdw)
        x_t.free_grad()
        return rdw

    dw = step(k_n)
    assert len(made) == 1                       # forward made it, the data gradient reused it
    nn.conv2D(x_t, k_t, stride=1).np()          # another geometry over the same kernel: same copy
    step(k_n)
    assert len(made) == 1
    opt.step()                                  # the weights change: the update writes the copy as well ...
    k2 = (k_n - 0.5 * dw).astype(np.float32)
    step(k2)
    assert len(made) == 1                       # ... so no permutation launch follows, and the passes above were exact
    k_t.set(k_n)
    step(k_n)
    assert len(made) == 2
    k_t.fill(1.0)
    step(np.ones_like(k_n))
    assert len(made) == 3
    k_t.np()                                    # reading does not invalidate
    step(np.ones_like(k_n))
    assert len(made) == 3
    # ... nor do operators that only read the kernel (a weight-decay term, a norm, a transposed view of it)
    nn.square(k_t).np()
    nn.reduce_sum(k_t).np()
    nn.transpose(k_t, (1, 0, 2, 3)).np()
    nn.mul(k_t, k_t).np()
    nn.add(k_t, nn.Tensor_from_value(np.ones((1,), np.float32))).np()
    step(np.ones_like(k_n))
    assert len(made) == 3


def test_transposed_convolution_copy_survives_optimizer_steps(nn_backend, monkeypatch):
    """The kernel of a transposed convolution is stored with swapped channel axes relative to the convolution whose
    passes it borrows; its permuted copy is made straight from that storage once, and SGD and Adam steps write the
    new values into it: no further permutation launch, and forward, input gradient and kernel gradient stay exact
    on the updated kernel."""
    nn = nn_backend
    from litenn_amd.core.hip import api
    made = []
    real = api.conv2d_permute_weights
    monkeypatch.setattr(api, 'conv2d_permute_weights', lambda *a: (made.append(1), real(*a))[1])
    rs = np.random.RandomState(12)
    for opt_name in ('sgd', 'adam'):
        made.clear()
        x_n = rs.randint(-2, 3, size=(2, 32, 5, 6)).astype(np.float32)
        k_n = rs.randint(-2, 3, size=(32, 32, 3, 3)).astype(np.float32)
        x_t, k_t = nn.Tensor_from_value(x_n), nn.Tensor_from_value(k_n)
        opt = nn.optimizer.SGD([k_t], lr=0.5) if opt_name == 'sgd' else nn.optimizer.Adam([k_t], lr=0.25)

        def step(expect_k, exact):
            y = nn.conv2DTranspose(x_t, k_t, stride=2)
            g_n = np.ones(tuple(y.shape), np.float32)
            ry, rdi, rdk = conv2d_transpose_all(x_n, expect_k, g_n, 2, 1, 'same')
            opt.zero_grad()
            nn.backward({y: g_n}, grad_for_non_trainables=True)
            if exact:
                assert np.array_equal(y.np(), ry) and np.array_equal(x_t.get_grad().np(), rdi)
                assert np.array_equal(k_t.get_grad().np(), rdk)
            else:
                # Adam's quotient m / (sqrt(v) + eps) is rounded differently on host and device; a copy that had
                # missed the step would be off by 0.25 per weight, i.e. by units in every output
                assert np.allclose(y.np(), ry, rtol=1e-3, atol=2e-2) and np.allclose(x_t.get_grad().np(), rdi, rtol=1e-3, atol=2e-2)
            x_t.free_grad()
            return rdk

        dk = step(k_n, True)
        assert len(made) == 1
        opt.step()
        if opt_name == 'sgd':
            k2 = (k_n - 0.5 * dk).astype(np.float32)
        else:   # first Adam step from zero moments: m = 0.1 g, v = 0.001 g^2
            m, v = np.float32(0.1) * dk, np.float32(0.001) * dk * dk
            k2 = (k_n - np.float32(0.25) * m / (np.sqrt(v) + np.float32(1e-7))).astype(np.float32)
        step(k2, opt_name == 'sgd')
        assert len(made) == 1, opt_name


def test_conv2d_transpose_module_and_errors(nn_backend):
    nn = nn_backend
    rs = np.random.RandomState(2)
    w = rs.randint(4, size=(8, 4, 3, 3)).astype(np.float32)
    b = rs.randint(4, size=(8,)).astype(np.float32)
    module = nn.Conv2DTranspose(4, 8, 3, kernel_initializer=nn.initializer.NumpyArray(w),
                                bias_initializer=nn.initializer.NumpyArray(b))
    x_n = rs.randint(4, size=(2, 4, 8, 8)).astype(np.float32)
    x = nn.Tensor_from_value(x_n)
    y = module(x)
    assert tuple(y.shape) == (2, 8, 16, 16)
    ref, dI, dK = conv2d_transpose_all(x_n, w, np.ones((2, 8, 16, 16), np.float32), 2, 1, 'same')
    assert np.array_equal(y.np(), ref + b.reshape(1, -1, 1, 1))
    y.backward(grad_for_non_trainables=True)
    assert np.array_equal(x.get_grad().np(), dI)
    assert np.array_equal(module.kernel.get_grad().np(), dK)
    assert np.array_equal(module.bias.get_grad().np(), np.full((8,), 2 * 16 * 16, np.float32))
    with pytest.raises(ValueError):
        nn.conv2DTranspose(x, module.kernel, padding=1)
    with pytest.raises(ValueError):
        nn.conv2DTranspose(x, nn.Tensor((8, 5, 3, 3)))


def test_conv2d_bias_act_equals_separate_ops(nn_backend):
    """The fused layer step leaky_relu(conv2D(x, k) + bias, alpha) must give the
    bits and the gradients of the three separate operators, on integer-valued
    data (alpha = 0.5 keeps every value exactly representable)."""
    nn = nn_backend
    import litenn_amd.core as nc
    rs = np.random.RandomState(4)
    for (n, ic, oc, hw, ks, stride, padding, alpha) in [(2, 3, 5, 9, 3, 1, 'same', 0.5), (1, 32, 40, 6, 3, 2, 1, 0.5),
                                                        (3, 4, 2, 8, 1, 1, 'valid', None), (1, 130, 70, 5, 3, 1, 'same', 0.25),
                                                        (2, 256, 96, 4, 3, 1, 'same', 0.5)]:
        x_n = rs.randint(-3, 4, size=(n, ic, hw, hw)).astype(np.float32)
        k_n = rs.randint(-3, 4, size=(oc, ic, ks, ks)).astype(np.float32)
        b_n = rs.randint(-9, 10, size=(oc,)).astype(np.float32)
        outs = []
        for fused in (False, True):
            x, k, b = nn.Tensor_from_value(x_n), nn.Tensor_from_value(k_n), nn.Tensor_from_value(b_n)
            if fused:
                y = nc.op.conv2D_bias_act(x, k, b, stride, 1, padding, leaky_relu_alpha=alpha)
            else:
                y = nn.conv2D(x, k, stride=stride, padding=padding) + b.reshape((1, -1, 1, 1))
                if alpha is not None:
                    y = nn.leaky_relu(y, alpha)
            g_n = np.random.RandomState(5).randint(-4, 5, size=tuple(y.shape)).astype(np.float32)
            nn.backward({y: g_n}, grad_for_non_trainables=True)
            outs.append((y.np(), x.get_grad().np(), k.get_grad().np(), b.get_grad().np()))
        for a, f in zip(*outs):
            assert np.array_equal(a, f), (n, ic, oc, hw, ks, stride, padding, alpha)
    with pytest.raises(ValueError):
        nc.op.conv2D_bias_act(nn.Tensor((1, 2, 4, 4)), nn.Tensor((3, 2, 3, 3)), nn.Tensor((4,)))
    with pytest.raises(ValueError):
        nc.op.conv2D_bias_act(nn.Tensor((1, 2, 4, 4)), nn.Tensor((3, 2, 3, 3)), leaky_relu_alpha=0.0)


def test_fused_epilogue_backward_twice_over_one_graph(nn_backend):
    """Two backward() sweeps over the same graph with grad_for_non_trainables=True accumulate: the output's own
    gradient holds 1x then 2x the seed (the same tensor object both times), so the second sweep adds twice the first
    sweep's contribution and every gradient of the fused node ends at three times a single sweep: its
    pre-activation gradient must be formed anew from the current dO in each sweep.  (The chain of three separate
    ops also keeps and re-propagates the gradients of its two intermediate tensors, so it is compared after the
    first sweep only.)"""
    nn = nn_backend
    import litenn_amd.core as nc
    rs = np.random.RandomState(12)
    x_n = rs.randint(-3, 4, size=(2, 3, 9, 9)).astype(np.float32)
    k_n = rs.randint(-3, 4, size=(4, 3, 3, 3)).astype(np.float32)
    b_n = rs.randint(-3, 4, size=(4,)).astype(np.float32)
    outs = []
    for fused in (False, True):
        x, k, b = nn.Tensor_from_value(x_n), nn.Tensor_from_value(k_n), nn.Tensor_from_value(b_n)
        if fused:
            y = nc.op.conv2D_bias_act(x, k, b, 1, 1, 'same', leaky_relu_alpha=0.5)
        else:
            y = nn.leaky_relu(nn.conv2D(x, k) + b.reshape((1, -1, 1, 1)), 0.5)
        g_n = np.random.RandomState(1).randint(-4, 5, size=tuple(y.shape)).astype(np.float32)
        nn.backward({y: g_n}, grad_for_non_trainables=True)
        once = (x.get_grad().np().copy(), k.get_grad().np().copy(), b.get_grad().np().copy())
        nn.backward({y: g_n}, grad_for_non_trainables=True)
        twice = (x.get_grad().np(), k.get_grad().np(), b.get_grad().np())
        if fused:
            for o, t in zip(once, twice):
                assert np.array_equal(t, 3 * o)
        outs.append(once)
        del x, k, b, y
    for a, f in zip(*outs):
        assert np.array_equal(a, f)


def test_fused_epilogue_lets_its_intermediate_go_with_its_last_reader(nn_backend, monkeypatch):
    """The pre-activation gradient the three gradient functions of a fused layer share is dropped when the last of
    them has run - before backward() moves on to the layer below - not when the whole sweep ends."""
    nn = nn_backend
    import litenn_amd.core as nc
    from litenn_amd.core.hip import api
    import importlib
    conv_mod = importlib.import_module('litenn_amd.core.op.conv2D')
    events = []
    real_bwd, real_drop = api.bias_act_bwd, conv_mod._EpilogueGrad._drop
    monkeypatch.setattr(api, 'bias_act_bwd', lambda *a: (events.append('bwd'), real_bwd(*a))[1])
    monkeypatch.setattr(conv_mod._EpilogueGrad, '_drop', lambda self: (events.append('drop'), real_drop(self))[1])
    rs = np.random.RandomState(3)
    x = nn.Tensor_from_value(rs.randint(-3, 4, size=(2, 3, 8, 8)).astype(np.float32))
    k1 = nn.Tensor_from_value(rs.randint(-3, 4, size=(4, 3, 3, 3)).astype(np.float32))
    k2 = nn.Tensor_from_value(rs.randint(-3, 4, size=(5, 4, 3, 3)).astype(np.float32))
    b1, b2 = nn.Tensor_from_value(np.ones((4,), np.float32)), nn.Tensor_from_value(np.ones((5,), np.float32))
    y = nc.op.conv2D_bias_act(x, k1, b1, 1, 1, 'same', leaky_relu_alpha=0.5)
    z = nc.op.conv2D_bias_act(y, k2, b2, 1, 1, 'same', leaky_relu_alpha=0.5)
    nn.backward({z: np.ones(tuple(z.shape), np.float32)}, grad_for_non_trainables=True)
    assert events == ['bwd', 'drop', 'bwd', 'drop']


def test_depthwise_conv2d_reference_style(nn_backend):
    """depthwise_conv2D_test (depthwise_conv2D.py:128-…): its grid of paddings,
    dilations, strides, kernel sizes and shapes, exact on integer-valued data,
    gradients accumulated onto a pre-filled 1.0."""
    nn = nn_backend
    rs = np.random.RandomState(6)
    n_cases = 0
    for padding, dilation, stride, ks in itertools.product(['same', 'valid', 0, 1, 2], [1, 2], [1, 2, 3], [1, 3, 5, 7]):
        for n, ic, hw in [(1, 1, 8), (4, 2, 16), (1, 4, 32)]:
            if padding == 'valid' and hw < (ks - 1) * dilation + 1:
                continue
            x_n = rs.randint(2 ** 4, size=(n, ic, hw, hw)).astype(np.float32)
            k_n = rs.randint(2 ** 4, size=(ic, ks, ks)).astype(np.float32)
            x, k = nn.Tensor_from_value(x_n), nn.Tensor_from_value(k_n)
            try:
                ci = info_conv2d(hw, hw, ks, ks, stride, dilation, padding)
            except ValueError:
                continue
            if ci.OH <= 0 or ci.OW <= 0:
                continue
            y = nn.depthwise_conv2D(x, k, stride=stride, dilation=dilation, padding=padding)
            g_n = rs.randint(2 ** 4, size=tuple(y.shape)).astype(np.float32)
            ry, rdi, rdk = depthwise_all(x_n, k_n, g_n, stride, dilation, padding)
            assert np.array_equal(y.np(), ry), (padding, dilation, stride, ks, n, ic, hw)
            x.get_grad().fill(1.0)
            k.get_grad().fill(1.0)
            nn.backward({y: g_n}, grad_for_non_trainables=True)
            assert np.array_equal(x.get_grad().np() - 1.0, rdi), (padding, dilation, stride, ks, n, ic, hw)
            assert np.array_equal(k.get_grad().np() - 1.0, rdk), (padding, dilation, stride, ks, n, ic, hw)
            n_cases += 1
    assert n_cases > 250


def test_depthwise_and_separable_modules(nn_backend):
    nn = nn_backend
    rs = np.random.RandomState(8)
    dk = rs.randint(-2, 3, size=(4, 3, 3)).astype(np.float32)
    pk = rs.randint(-2, 3, size=(6, 4, 1, 1)).astype(np.float32)
    b = rs.randint(-2, 3, size=(6,)).astype(np.float32)
    x_n = rs.randint(-2, 3, size=(2, 4, 8, 8)).astype(np.float32)
    sep = nn.SeparableConv2D(4, 6, 3, depthwise_initializer=nn.initializer.NumpyArray(dk),
                             pointwise_initializer=nn.initializer.NumpyArray(pk),
                             bias_initializer=nn.initializer.NumpyArray(b))
    x = nn.Tensor_from_value(x_n)
    y = sep(x)
    mid, _, _ = depthwise_all(x_n, dk, np.zeros((2, 4, 8, 8)), 1, 1, 'same')
    ref, _, _ = conv2d_all(mid, pk, np.zeros((2, 6, 8, 8)), 1, 1, 'valid')
    assert np.array_equal(y.np(), ref + b.reshape(1, -1, 1, 1))
    y.backward(grad_for_non_trainables=True)
    ones = np.ones((2, 6, 8, 8))
    _, dmid, dpk = conv2d_all(mid, pk, ones, 1, 1, 'valid')
    _, dx, ddk = depthwise_all(x_n, dk, dmid, 1, 1, 'same')
    assert np.array_equal(x.get_grad().np(), dx)
    assert np.array_equal(sep.depthwise_kernel.get_grad().np(), ddk)
    assert np.array_equal(sep.pointwise_kernel.get_grad().np(), dpk)
    assert np.array_equal(sep.bias.get_grad().np(), np.full((6,), 2 * 64, np.float32))
    dwm = nn.DepthwiseConv2D(4, 3, use_bias=False, depthwise_initializer=nn.initializer.NumpyArray(dk))
    y2 = dwm(nn.Tensor_from_value(x_n))
    assert np.array_equal(y2.np(), mid)
    with pytest.raises(ValueError):
        nn.depthwise_conv2D(x, nn.Tensor((4, 1, 3, 3)))
    with pytest.raises(ValueError):
        nn.depthwise_conv2D(x, nn.Tensor((5, 3, 3)))


def test_matmul_reference_style(nn_backend):
    nn = nn_backend
    rs = np.random.RandomState(1)
    for _ in range(10):
        BATCH, M = rs.randint(8) + 1, rs.randint(8) + 1
        N, K = rs.randint(32768) + 1, rs.randint(32768) + 1
        while K * N > (400000 // BATCH):
            K, N = max(1, K // 2), max(1, N // 2)
        if rs.randint(2) == 0:
            size = [2, 4, 8, 16][rs.randint(4)]
            M, N, K = (max(1, v // size) * size for v in (M, N, K))
        A_shape, B_shape = ((M, K), (K, N)) if BATCH == 1 else ((BATCH, M, K), (BATCH, K, N))
        A_n = rs.randint(2 ** 4, size=A_shape).astype(np.float32)
        B_n = rs.randint(2 ** 4, size=B_shape).astype(np.float32)
        O_n = np.matmul(A_n, B_n)
        A_t, B_t = nn.Tensor_from_value(A_n), nn.Tensor_from_value(B_n)
        O_t = nn.matmul(A_t, B_t)
        assert O_n.shape == O_t.shape
        assert np.array_equal(O_t.np(), O_n)
        O_n_grad = rs.randint(2 ** 3, size=O_n.shape).astype(np.float32)
        A_t.get_grad().fill(1.0)
        B_t.get_grad().fill(1.0)
        nn.backward({O_t: O_n_grad}, grad_for_non_trainables=True)
        assert np.array_equal(A_t.get_grad().np() - 1.0, np.matmul(O_n_grad, np.swapaxes(B_n, -1, -2)))
        assert np.array_equal(B_t.get_grad().np() - 1.0, np.matmul(np.swapaxes(A_n, -1, -2), O_n_grad))


def test_matmul_and_conv_shape_errors(nn_backend):
    nn = nn_backend
    with pytest.raises(ValueError):
        nn.matmul(nn.Tensor((2, 3)), nn.Tensor((1, 3, 4)))
    with pytest.raises(ValueError):
        nn.matmul(nn.Tensor((3,)), nn.Tensor((3,)))
    with pytest.raises(ValueError):
        nn.matmul(nn.Tensor((2, 3)), nn.Tensor((4, 5)))
    with pytest.raises(ValueError):
        nn.matmul(nn.Tensor((2, 2, 3)), nn.Tensor((3, 3, 4)))
    with pytest.raises(ValueError):
        nn.conv2D(nn.Tensor((1, 3, 4, 4)), nn.Tensor((2, 4, 3, 3)))
    with pytest.raises(ValueError):
        nn.conv2D(nn.Tensor((1, 3, 4, 4)), nn.Tensor((2, 3, 3, 3)), padding='full')
    with pytest.raises(ValueError):
        nn.conv2D(nn.Tensor((1, 3, 4, 4)), nn.Tensor((2, 3, 3, 3)), padding=(1, 2, 3))


def test_output_t_and_is_add_to_output(nn_backend):
    nn = nn_backend
    import litenn_amd.core as nc
    rs = np.random.RandomState(2)
    a = rs.randint(8, size=(6, 5)).astype(np.float32)
    b = rs.randint(8, size=(5, 7)).astype(np.float32)
    a_t, b_t = nn.Tensor_from_value(a), nn.Tensor_from_value(b)
    out = nn.Tensor((42,), init=nn.initializer.Scalar(3.0))          # any shape of equal size
    r = nc.op.matmul(a_t, b_t, output_t=out, is_add_to_output=True)
    assert r is out and not out._is_produced_by_op()
    assert np.array_equal(out.np().reshape(6, 7), a @ b + 3.0)
    nc.op.matmul(a_t, b_t, output_t=out)                             # overwrite
    assert np.array_equal(out.np().reshape(6, 7), a @ b)
    with pytest.raises(ValueError):
        nc.op.matmul(a_t, b_t, output_t=nn.Tensor((41,)))
    t = nn.Tensor((7, 6), init=nn.initializer.Scalar(1.0))
    nc.op.transpose(nn.Tensor_from_value(a @ b), (1, 0), output_t=t, is_add_to_output=True)
    assert np.array_equal(t.np(), (a @ b).T + 1.0)


def test_transpose_reference_style(nn_backend):
    nn = nn_backend
    rs = np.random.RandomState(3)
    for _ in range(5):
        for rank in range(2, 5):
            shape = rs.randint(8, size=(rank,)) + 1
            axes = rs.permutation(rank)
            val_n = rs.randint(2 ** 8, size=shape).astype(np.float32)
            val_t = nn.Tensor_from_value(val_n)
            tr_t = nn.transpose(val_t, axes)
            assert np.array_equal(tr_t.np(), np.transpose(val_n, axes))
            g = rs.randint(2 ** 8, size=tuple(tr_t.shape)).astype(np.float32)
            val_t.get_grad().fill(1.0)
            nn.backward({tr_t: g}, grad_for_non_trainables=True)
            assert np.array_equal(np.transpose(val_t.get_grad().np() - 1.0, axes), g)
    for size in (2, 3):
        v = rs.randint(2 ** 8, size=(2, 2 * size * size, 3 * size, 3 * size)).astype(np.float32)
        v_t = nn.Tensor_from_value(v)
        assert np.array_equal(nn.space_to_depth(nn.depth_to_space(v_t, size), size).np(), v)


def test_reshape_is_a_view(nn_backend):
    nn = nn_backend
    v = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    t = nn.Tensor_from_value(v)
    r = t.reshape((4, -1))
    assert r._is_reference() and r.shape == (4, 6)
    assert np.array_equal(r.np(), v.reshape(4, 6))
    r.set(np.ones((4, 6)))
    assert np.array_equal(t.np(), np.ones((2, 3, 4)))                 # same storage
    assert nn.flatten(t).shape == (2, 12)
    with pytest.raises(ValueError):
        t.reshape((5, -1))
    g = r.get_grad()
    assert t.has_grad() and g.shape == (4, 6)


def test_backward_freeze_and_optimizer(nn_backend):
    nn = nn_backend
    inp_t = nn.Tensor((2, 2, 8, 8), init=nn.initializer.Scalar(1.0))
    kernel_t = nn.Tensor((4, 2, 3, 3), init=nn.initializer.Scalar(0.0))
    kernel_2_t = nn.Tensor((4, 2, 3, 3), init=nn.initializer.Scalar(0.0))
    opt = nn.optimizer.SGD([inp_t, kernel_t, kernel_2_t])
    opt.zero_grad()
    with nn.optimizer.freeze():
        r = nn.conv2D(inp_t, kernel_2_t)
    r.backward()
    assert not kernel_2_t.has_grad()
    r = nn.conv2D(inp_t, kernel_t)
    r.backward()
    assert kernel_t.has_grad()
    assert not np.all(kernel_t.get_grad().np() == 0)
    opt.step()
    assert not np.all(kernel_t.np() == 0)
    assert opt.get_iteration() == 1


def test_non_trainable_gradients_are_dropped(nn_backend):
    nn = nn_backend
    x = nn.Tensor_from_value(np.ones((1, 2, 4, 4), np.float32))
    w = nn.Tensor_from_value(np.ones((3, 2, 3, 3), np.float32))
    y = nn.leaky_relu(nn.conv2D(x, w))
    y.backward()                                   # nothing is attached to an optimizer
    assert not x.has_grad() and not w.has_grad() and not y.has_grad()
    y.backward(grad_for_non_trainables=True)
    assert x.has_grad() and w.has_grad() and y.has_grad()
    x.free_grad(); w.free_grad()
    opt = nn.optimizer.SGD([w])
    y2 = nn.leaky_relu(nn.conv2D(x, w))
    y2.backward()
    assert w.has_grad() and not x.has_grad() and not y2.has_grad()   # only the trainable keeps its grad
    w.zero_grad()
    y3 = nn.conv2D(x, w)
    y3.backward(stop_grad=[y3])
    assert not w.has_grad()
    del opt


def test_conv2d_and_dense_modules(nn_backend):
    nn = nn_backend
    module = nn.Conv2D(4, 8, 3)
    x = nn.Tensor((2, 4, 8, 8))
    y = module(x)
    y.backward(grad_for_non_trainables=True)
    assert x.has_grad() and y.shape == (2, 8, 8, 8)
    assert [t.get_name() for t in module.trainables()] == ['Conv2D.kernel', 'Conv2D.bias']
    dense = nn.Dense(4, 8)
    x2 = nn.Tensor((2, 4))
    y2 = dense(x2)
    y2.backward(grad_for_non_trainables=True)
    assert x2.has_grad() and y2.shape == (2, 8)
    # numeric check with a bias
    rs = np.random.RandomState(4)
    k = rs.randint(4, size=(5, 3, 3, 3)).astype(np.float32)
    b = rs.randint(4, size=(5,)).astype(np.float32)
    conv = nn.Conv2D(3, 5, 3, stride=2, kernel_initializer=nn.initializer.NumpyArray(k),
                     bias_initializer=nn.initializer.NumpyArray(b))
    xv = rs.randint(4, size=(2, 3, 9, 9)).astype(np.float32)
    out = conv(nn.Tensor_from_value(xv))
    ci = info_conv2d(9, 9, 3, 3, 2, 1, 'same')
    gy = rs.randint(4, size=(2, 5, ci.OH, ci.OW)).astype(np.float32)
    ry, rdx, rdw = conv2d_all(xv, k, gy, 2, 1, 'same')
    assert np.array_equal(out.np(), ry + b.reshape(1, 5, 1, 1))
    nn.backward({out: gy}, grad_for_non_trainables=True)
    assert np.array_equal(conv.kernel.get_grad().np(), rdw)
    assert np.array_equal(conv.bias.get_grad().np(), gy.sum((0, 2, 3)))


def test_dense_bias_in_the_product_epilogue(nn_backend):
    """Dense.forward = nn.matmul(x, weight) + bias (module/Dense.py:44-48) with the bias added by the product's
    epilogue: same values and same gradients as the two separate ops, also behind an activation and when the
    gradients already hold something."""
    import litenn_amd.core as nc
    nn = nn_backend
    rs = np.random.RandomState(8)
    for rows, n_in, n_out in ((5, 12, 20), (32, 64, 256), (70, 16, 8)):
        w = rs.randint(-4, 5, size=(n_in, n_out)).astype(np.float32)
        b = rs.randint(-4, 5, size=(n_out,)).astype(np.float32)
        xv = rs.randint(-4, 5, size=(rows, n_in)).astype(np.float32)
        gy = rs.randint(-4, 5, size=(rows, n_out)).astype(np.float32)
        dense = nn.Dense(n_in, n_out, weight_initializer=nn.initializer.NumpyArray(w),
                         bias_initializer=nn.initializer.NumpyArray(b))
        x = nn.Tensor_from_value(xv)
        y = dense(x)
        assert y.shape == (rows, n_out)
        want = xv.astype(np.float64) @ w + b
        assert np.array_equal(y.np(), want)
        nn.backward({y: gy}, grad_for_non_trainables=True)
        assert np.array_equal(x.get_grad().np(), gy.astype(np.float64) @ w.T)
        assert np.array_equal(dense.weight.get_grad().np(), xv.T.astype(np.float64) @ gy)
        assert np.array_equal(dense.bias.get_grad().np(), gy.sum(0))
        # a second sweep accumulates into the same gradients
        y = dense(x)
        nn.backward({y: gy}, grad_for_non_trainables=True)
        assert np.array_equal(dense.bias.get_grad().np(), 2 * gy.sum(0))
        assert np.array_equal(dense.weight.get_grad().np(), 2 * (xv.T.astype(np.float64) @ gy))
        # the fused activation: leaky_relu(x @ w + b)
        x2, w2, b2 = nn.Tensor_from_value(xv), nn.Tensor_from_value(w), nn.Tensor_from_value(b)
        z = nc.op.matmul_bias_act(x2, w2, b2, leaky_relu_alpha=0.5)
        pre = want
        assert np.array_equal(z.np(), np.where(pre >= 0, pre, 0.5 * pre))
        nn.backward({z: gy}, grad_for_non_trainables=True)
        dpre = gy * np.where(pre >= 0, 1.0, 0.5)
        assert np.array_equal(b2.get_grad().np(), dpre.sum(0))
        assert np.array_equal(w2.get_grad().np(), xv.T.astype(np.float64) @ dpre)
        assert np.array_equal(x2.get_grad().np(), dpre @ w.T.astype(np.float64))
    with pytest.raises(ValueError):
        nc.op.matmul_bias_act(nn.Tensor((4, 6)), nn.Tensor((6, 8)), nn.Tensor((7,)))
    with pytest.raises(ValueError):
        nc.op.matmul_bias_act(nn.Tensor((4, 6)), nn.Tensor((6, 8)), None, leaky_relu_alpha=0.0)


def test_shallow_mode_allocates_nothing(nn_backend):
    nn = nn_backend

    class M(nn.Module):
        def __init__(self):
            self.conv = nn.Conv2D(1, 1, 3, stride=2)

        def forward(self, x):
            return self.conv(x)

    m = M()
    m.set_training(True)
    out = m.shallow_forward(nn.Tensor((1, 1, 16, 16)))
    assert out.shape == (1, 1, 8, 8)
    assert nn.devices.get_current()[0].get_used_memory() == 0
    assert m.is_training() and m.conv.is_training()


def test_sgd_closed_form(nn_backend):
    nn = nn_backend
    for momentum, nesterov, decay in [(0.0, False, 0.0), (0.9, False, 0.0), (0.9, True, 0.1)]:
        w0 = np.linspace(-1, 1, 16).astype(np.float32)
        g = np.linspace(1, 2, 16).astype(np.float32)
        w_t = nn.Tensor_from_value(w0)
        opt = nn.optimizer.SGD([w_t], momentum=momentum, nesterov=nesterov, lr=0.01, lr_decay=decay)
        w, acc = w0.astype(np.float64), np.zeros(16)
        for it in range(3):
            w_t.get_grad().set(g)
            opt.step()
            lr = 0.01 / (1.0 + decay * it)
            acc = momentum * acc - lr * g
            w = w + (momentum * acc - lr * g if nesterov else acc)
        np.testing.assert_allclose(w_t.np(), w, rtol=1e-5, atol=1e-6)
        w_t._set_trainable(False)
    with pytest.raises(ValueError):
        nn.optimizer.SGD([nn.Tensor((4,))], lr_dropout=1.7)


def test_lr_dropout_follows_the_counter_hash(nn_backend):
    """Optimizer.py:178-203: every update kernel draws a seed from numpy's global generator and zeroes the learning
    rate of element gid where hash_float_uint(gid + seed) <= lr_dropout.  With the generator seeded, the dropped
    elements are those the oracle's hash names, for SGD (two kernels per tensor, SGD.py:42-83) and Adam (one,
    Adam.py:61-86)."""
    nn = nn_backend
    n, p = 5000, 0.3
    rs = np.random.RandomState(2)
    w0 = rs.randint(-8, 9, size=n).astype(np.float32)
    g = rs.randint(1, 9, size=n).astype(np.float32)
    for nesterov in (False, True):
        w_t = nn.Tensor_from_value(w0)
        opt = nn.optimizer.SGD([w_t], momentum=0.5, nesterov=nesterov, lr=0.25, lr_dropout=p)
        np.random.seed(77)
        seeds = [int(np.random.randint(2147483648)) for _ in range(4)]
        np.random.seed(77)
        w, acc = w0.astype(np.float64), np.zeros(n)
        for it in range(2):
            w_t.get_grad().set(g)
            opt.step()
            lr_a = np.where(hash_rng.lr_dropout_mask(n, seeds[2 * it], p), 0.0, 0.25)
            lr_t = np.where(hash_rng.lr_dropout_mask(n, seeds[2 * it + 1], p), 0.0, 0.25)
            acc = 0.5 * acc - lr_a * g
            w = w + (0.5 * acc - lr_t * g if nesterov else acc)
        assert np.array_equal(w_t.np(), w)          # small integers and quarters: exact in fp32
        assert 0.2 < hash_rng.lr_dropout_mask(n, seeds[0], p).mean() < 0.4
        w_t._set_trainable(False)
    w_t = nn.Tensor_from_value(w0)
    opt = nn.optimizer.Adam([w_t], lr=0.5, lr_dropout=p)
    np.random.seed(78)
    seed = int(np.random.randint(2147483648))
    np.random.seed(78)
    w_t.get_grad().set(g)
    opt.step()
    dropped = hash_rng.lr_dropout_mask(n, seed, p)
    got = w_t.np()
    assert np.array_equal(got[dropped], w0[dropped]) and np.all(got[~dropped] != w0[~dropped])
    w_t._set_trainable(False)
    # the seeds are drawn whether or not dropout is on, as the reference does: the generator stays in step with it
    w_t = nn.Tensor_from_value(w0)
    opt = nn.optimizer.SGD([w_t], lr=0.25)
    np.random.seed(79)
    expect = np.random.RandomState(79)
    w_t.get_grad().set(g)
    opt.step()
    expect.randint(2147483648), expect.randint(2147483648)
    assert np.random.randint(1 << 30) == expect.randint(1 << 30)
    w_t._set_trainable(False)


def test_adam_closed_form(nn_backend):
    """Adam.py:43-72 in float64: m and v without bias correction, t += -lr*m/(sqrt(v)+1e-7)."""
    nn = nn_backend
    for b1, b2, decay in [(0.9, 0.999, 0.0), (0.5, 0.9, 0.1)]:
        w0 = np.linspace(-1, 1, 37).astype(np.float32)
        w_t = nn.Tensor_from_value(w0)
        opt = nn.optimizer.Adam([w_t], beta_1=b1, beta_2=b2, lr=0.01, lr_decay=decay)
        w, m, v = w0.astype(np.float64), np.zeros(37), np.zeros(37)
        for it in range(4):
            g = np.linspace(1 + it, 2, 37).astype(np.float32) * (-1) ** it
            w_t.get_grad().set(g)
            opt.step()
            lr = 0.01 / (1.0 + decay * it)
            m = b1 * m + (1 - b1) * g
            v = b2 * v + (1 - b2) * g.astype(np.float64) ** 2
            w = w - lr * m / (np.sqrt(v) + 1e-7)
        np.testing.assert_allclose(w_t.np(), w, rtol=2e-5, atol=1e-6)
        w_t._set_trainable(False)


def test_random_initializers_fill_on_device(nn_backend):
    """InitRandomUniform_test / InitRandomNormal_test and the He / Glorot lines of the reference's own test
    (test.py:237-242), plus what the seed draw promises: np.random.seed fixes the weights, and they equal the
    counter-hash stream of that seed (initializer/RandomUniform.py:17-27, RandomNormal.py:14-30)."""
    nn = nn_backend
    for init in [nn.initializer.GlorotUniform(1.0, 1.0, 1.0), nn.initializer.GlorotNormal(1.0, 1.0, 1.0),
                 nn.initializer.HeUniform(1.0, 1.0), nn.initializer.HeNormal(1.0, 1.0),
                 nn.initializer.RandomNormal(), nn.initializer.RandomUniform()]:
        v = nn.Tensor((128,), init=init).np()
        assert v.shape == (128,) and np.isfinite(v).all() and v.std() > 0.05

    def seeds(k, n):
        np.random.seed(k)
        return [int(np.random.randint(2147483648)) for _ in range(n)]

    np.random.seed(5)
    u = nn.Tensor((3, 1000), init=nn.initializer.RandomUniform(-0.5, 1.5)).np()
    z = nn.Tensor((4096,), init=nn.initializer.RandomNormal(0.25, 2.0)).np()
    s0, s1 = seeds(5, 2)
    assert np.allclose(u.reshape(-1), hash_rng.random_uniform(3000, s0, -0.5, 1.5), rtol=0, atol=3e-7)
    assert np.allclose(z, hash_rng.random_normal(4096, s1, 0.25, 2.0), rtol=0, atol=2e-5)
    assert u.min() >= -0.5 and u.max() <= 1.5

    # default construction of the layers draws their kernels on the device, each with its own bound
    np.random.seed(11)
    conv = nn.Conv2D(8, 16, 3)
    dense = nn.Dense(32, 64)
    k, w = conv.kernel.np(), dense.weight.np()
    a_conv = np.sqrt(3.0) * np.sqrt(2.0 / (8 * 9 + 16 * 9))
    a_dense = np.sqrt(3.0) * np.sqrt(2.0 / (32 + 64))
    assert np.abs(k).max() <= a_conv and np.abs(k).max() > 0.9 * a_conv
    assert np.abs(w).max() <= a_dense and np.abs(w).max() > 0.9 * a_dense
    s0 = seeds(11, 1)[0]
    assert np.allclose(k.reshape(-1), hash_rng.random_uniform(k.size, s0, -a_conv, a_conv), rtol=0, atol=1e-7)
    np.random.seed(11)
    assert np.array_equal(nn.Conv2D(8, 16, 3).kernel.np(), k)

    with pytest.raises(ValueError):
        nn.Tensor((4,), init=nn.initializer.HeNormal()).np()          # fan_in never set
    with pytest.raises(ValueError):
        nn.Tensor((4,), init=nn.initializer.GlorotUniform(fan_in=3)).np()


def test_pointwise_broadcast_and_reduce(nn_backend):
    nn = nn_backend
    rs = np.random.RandomState(5)
    a = rs.randint(-8, 8, size=(2, 3, 4, 5)).astype(np.float32)
    b = rs.randint(-8, 8, size=(1, 3, 1, 1)).astype(np.float32)
    a_t, b_t = nn.Tensor_from_value(a), nn.Tensor_from_value(b)
    s = a_t + b_t
    assert np.array_equal(s.np(), a + b)
    m = a_t * b_t
    assert np.array_equal(m.np(), a * b)
    d = a_t - b_t
    g = rs.randint(-4, 4, size=(2, 3, 4, 5)).astype(np.float32)
    nn.backward({s: g, m: g, d: g}, grad_for_non_trainables=True)
    assert np.array_equal(a_t.get_grad().np(), g + g * b + g)
    assert np.array_equal(b_t.get_grad().np(), (g + g * a - g).sum((0, 2, 3), keepdims=True))
    a_t.free_grad()
    lr = nn.leaky_relu(a_t, 0.5)
    assert np.array_equal(lr.np(), np.where(a >= 0, a, 0.5 * a))
    sq = nn.square(a_t)
    mean = sq.mean()
    assert mean.shape == (1,)
    np.testing.assert_allclose(mean.np()[0], (a * a).mean(), rtol=1e-6)
    nn.backward([mean], grad_for_non_trainables=True)
    np.testing.assert_allclose(a_t.get_grad().np(), 2 * a / a.size, rtol=1e-6)
    r = nn.reduce_sum(a_t, axes=(1, -1), keepdims=True)
    assert r.shape == (2, 1, 4, 1) and np.array_equal(r.np(), a.sum((1, 3), keepdims=True))
    r2 = a_t.sum(axes=0)
    assert r2.shape == (3, 4, 5) and np.array_equal(r2.np(), a.sum(0))
    assert np.array_equal((a_t + 2).np(), a + 2) and np.array_equal((3 * a_t).np(), 3 * a)
    assert np.array_equal((a_t + a_t).np(), 2 * a) and np.array_equal((-a_t).np(), -a)


def test_buffer_pool_and_lifetime_guards(nn_backend):
    nn = nn_backend
    dev = nn.devices.get_current()[0]
    t = nn.Tensor((256,))
    assert dev.get_used_memory() == 0                       # allocation is lazy
    t.np()
    assert dev.get_used_memory() == 1024
    del t
    assert dev.get_used_memory() == 0 and dev.get_total_pooled_memory() == 1024
    t2 = nn.Tensor((256,), init=nn.initializer.Scalar(2.0))
    assert np.array_equal(t2.np(), np.full(256, 2.0, np.float32))     # pooled block is re-initialised
    assert dev.get_total_allocated_memory() == 1024
    with pytest.raises(Exception):
        nn.cleanup()                                         # a Tensor is alive
    with pytest.raises(Exception):
        nn.devices.set_current(dev)
    del t2
    nn.cleanup()
    assert dev.get_total_allocated_memory() == 0


def test_module_names_save_and_load(nn_backend, tmp_path):
    nn = nn_backend

    class Net(nn.Module):
        def __init__(self):
            self.blocks = [nn.Conv2D(2, 2, 3), nn.Conv2D(2, 2, 1, use_bias=False)]
            self.head = nn.Dense(8, 3)
            self.note = 'v1'

        def forward(self, x):
            for b in self.blocks:
                x = b(x)
            return self.head(nn.flatten(x))

    net = Net()
    names = [t.get_name() for t in net.trainables()]
    assert names == ['Net.blocks[0].kernel', 'Net.blocks[0].bias', 'Net.blocks[1].kernel', 'Net.head.weight',
                     'Net.head.bias']
    assert net(nn.Tensor((1, 2, 2, 2))).shape == (1, 3)
    opt = nn.optimizer.SGD(net.trainables(), momentum=0.5)
    before = net.blocks[0].kernel.np().copy()
    path = tmp_path / 'net.bin'
    net.save(path)
    net.blocks[0].kernel.fill(7.0)
    net.note = 'changed'
    assert net.load(path) is True
    assert np.array_equal(net.blocks[0].kernel.np(), before) and net.note == 'v1'
    assert net.load(tmp_path / 'missing.bin') is False
    opt.iteration = 5
    opt.save(tmp_path / 'opt.bin')
    opt.iteration = 0
    opt.load(tmp_path / 'opt.bin')
    assert opt.iteration == 5
    with pytest.raises(ValueError):
        nn.optimizer.SGD(net.trainables())                  # already attached


def test_state_dict_has_the_reference_layout(nn_backend, caplog):
    """dump_state() / load_state() use the flat layout of ModuleBase.py:131-199, so checkpoints are
    interchangeable with the reference: tensors under '<path>.<attr>' as ('np.ndarray', array) - '.attr' with the
    leading dot for a tensor of the saved module itself -, python values as ('python-var', (class name, value)),
    list lengths as a bare int under '<name>__len', dict elements under '<name>[key]'.  The expected dict below is
    written out by hand from that layout, not produced by this package."""
    nn = nn_backend

    class Net(nn.Module):
        def __init__(self):
            self.blocks = [nn.Conv2D(2, 2, 3), nn.Conv2D(2, 2, 1, use_bias=False)]
            self.head = nn.Dense(8, 3)
            self.note = 'v1'
            self.scale = nn.Tensor((2,), init=nn.initializer.Scalar(1.0))
            self.d = {'a': 3, 'b': [1.5, 'x']}
            self.flag = True
            self.tup = (1, 2)            # tuples, None and arrays are not part of the state
            self.nothing = None
            self._hidden = 5             # underscore names are skipped unless listed as saveable

    net = Net()
    state = net.dump_state()
    expect_vars = {'blocks__len': 2, 'note': ('python-var', ('str', 'v1')), 'd[a]': ('python-var', ('int', 3)),
                   'd[b]__len': 2, 'd[b][0]': ('python-var', ('float', 1.5)), 'd[b][1]': ('python-var', ('str', 'x')),
                   'flag': ('python-var', ('bool', True))}
    expect_tensors = {'blocks[0].kernel': (2, 2, 3, 3), 'blocks[0].bias': (2,), 'blocks[1].kernel': (2, 2, 1, 1),
                      'head.weight': (8, 3), 'head.bias': (3,), '.scale': (2,)}
    assert set(state) == set(expect_vars) | set(expect_tensors)
    for k, v in expect_vars.items():
        assert state[k] == v and type(state[k]) is type(v), k
    for k, shape in expect_tensors.items():
        kind, arr = state[k]
        assert kind == 'np.ndarray' and isinstance(arr, np.ndarray) and arr.shape == shape and arr.dtype == np.float32, k

    # a state dict as the reference would have written it for the same model
    rs = np.random.RandomState(3)
    ref_state = {k: ('np.ndarray', rs.normal(0, 1, shape).astype(np.float32)) for k, shape in expect_tensors.items()}
    ref_state.update({'blocks__len': 2, 'note': ('python-var', ('str', 'from-reference')),
                      'd[a]': ('python-var', ('int', 11)), 'd[b]__len': 2, 'd[b][0]': ('python-var', ('float', 2.5)),
                      'd[b][1]': ('python-var', ('str', 'y')), 'flag': ('python-var', ('bool', False))})
    net.load_state(ref_state)
    assert net.note == 'from-reference' and net.d == {'a': 11, 'b': [2.5, 'y']} and net.flag is False
    assert np.array_equal(net.blocks[1].kernel.np(), ref_state['blocks[1].kernel'][1])
    assert np.array_equal(net.scale.np(), ref_state['.scale'][1])
    assert np.array_equal(net.head.weight.np(), ref_state['head.weight'][1])

    # mismatches warn and leave the value alone: class name, tensor shape, kind, list length (elements skipped too)
    caplog.clear()
    bad = dict(ref_state)
    bad['note'] = ('python-var', ('int', 7))
    bad['d[a]'] = ('np.ndarray', np.zeros(1, np.float32))
    bad['head.bias'] = ('np.ndarray', np.zeros((4,), np.float32))
    bad['d[b]__len'] = 3
    bad['d[b][0]'] = ('python-var', ('float', 99.0))
    del bad['flag']
    with caplog.at_level('WARNING', logger='litenn'):
        net.load_state(bad)
    assert net.note == 'from-reference' and net.d == {'a': 11, 'b': [2.5, 'y']} and net.flag is False
    assert np.array_equal(net.head.bias.np(), ref_state['head.bias'][1])
    text = caplog.text
    for needle in ('note', 'd[a]', 'head.bias', 'List d[b]', 'flag'):
        assert needle in text, needle

    # optimizers: the iteration counter and the accumulators, keyed by the tensors' full names
    opt = nn.optimizer.SGD(net.trainables(), momentum=0.5)
    ostate = opt.dump_state()
    assert ostate['iteration'] == ('python-var', ('int', 0))
    assert set(ostate) == {'iteration'} | {f'._accs[{t.get_name()}]' for t in net.trainables()}
    assert '._accs[Net.blocks[0].kernel]' in ostate
    ostate['iteration'] = ('python-var', ('int', 41))
    acc = np.full((2, 2, 3, 3), 0.25, np.float32)
    ostate['._accs[Net.blocks[0].kernel]'] = ('np.ndarray', acc)
    opt.load_state(ostate)
    assert opt.iteration == 41 and isinstance(opt.iteration, int)
    assert np.array_equal(opt._accs['Net.blocks[0].kernel'].np(), acc)


def test_library_side_out_of_memory_evicts_pooled_blocks(nn_backend):
    """A library call that reports out-of-memory for its own scratch is repeated after a pooled (idle) block has
    been released, largest first, like a failed tensor allocation (CLDevice.py:134-164); with an empty pool the
    error surfaces."""
    nn = nn_backend
    from litenn_amd.core.hip import api, launch
    dev = nn.devices.get_current()[0]
    for n in (1000, 3000, 2000):
        nn.Tensor((n,)).np()                      # allocate, then drop: the blocks go to the pool
    assert dev._total_buffers_pooled == 3
    t = nn.Tensor_from_value(np.arange(4, dtype=np.float32))
    calls = []

    def scratch_hungry(device_index, ptr):
        calls.append(dev._total_memory_pooled)
        if len(calls) <= 2:
            raise api.HipException(api.ERR_OOM, 'out of device memory for scratch')

    launch(scratch_hungry, t)
    assert calls == [24000, 12000, 4000]          # 3000 floats released first, then 2000
    assert dev._total_buffers_pooled == 1

    def always(device_index, ptr):
        raise api.HipException(api.ERR_OOM, 'out of device memory for scratch')
    with pytest.raises(api.HipException) as e:
        launch(always, t)
    assert e.value.code == api.ERR_OOM and dev._total_buffers_pooled == 0

    def other(device_index, ptr):
        raise api.HipException(api.ERR_INVALID, 'bad argument')
    nn.Tensor((500,)).np()
    with pytest.raises(api.HipException):
        launch(other, t)
    assert dev._total_buffers_pooled == 1         # other errors do not touch the pool
    del t


def test_training_step_matches_numpy(nn_backend):
    """Two-layer version of the encoder benchmark: conv(5x5, s2, p2) + bias ->
    leaky_relu(0.1) -> conv -> mean(square); SGD.  Compared with a float64
    restatement built from the oracle."""
    nn = nn_backend
    rs = np.random.RandomState(0)
    x = rs.uniform(-1, 1, (4, 3, 16, 16)).astype(np.float32)
    w1 = rs.normal(0, np.sqrt(2 / 75), (8, 3, 5, 5)).astype(np.float32)
    w2 = rs.normal(0, np.sqrt(2 / 200), (16, 8, 5, 5)).astype(np.float32)
    c1 = nn.Conv2D(3, 8, 5, stride=2, padding=2, kernel_initializer=nn.initializer.NumpyArray(w1))
    c2 = nn.Conv2D(8, 16, 5, stride=2, padding=2, kernel_initializer=nn.initializer.NumpyArray(w2))

    class A(nn.Module):
        def __init__(self): self.c1 = c1
    class B(nn.Module):
        def __init__(self): self.c2 = c2
    ma, mb = A(), B()
    opt = nn.optimizer.SGD(ma.trainables() + mb.trainables(), lr=1e-2)
    x_t = nn.Tensor_from_value(x)
    losses = []
    W1, W2 = w1.astype(np.float64), w2.astype(np.float64)
    B1, B2 = np.zeros(8), np.zeros(16)
    from oracle import conv2d_fwd, conv2d_dx, conv2d_dw
    for _ in range(2):
        opt.zero_grad()
        loss = nn.square(c2(nn.leaky_relu(c1(x_t), 0.1))).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.np()[0]))
        # float64 restatement
        z1 = conv2d_fwd(x, W1, 2, 1, 2) + B1.reshape(1, -1, 1, 1)
        a1 = np.where(z1 >= 0, z1, 0.1 * z1)
        z2 = conv2d_fwd(a1, W2, 2, 1, 2) + B2.reshape(1, -1, 1, 1)
        ref_loss = (z2 * z2).mean()
        dz2 = 2 * z2 / z2.size
        dW2, dB2 = conv2d_dw(a1, dz2, W2.shape, 2, 1, 2), dz2.sum((0, 2, 3))
        da1 = conv2d_dx(dz2, W2, a1.shape, 2, 1, 2)
        dz1 = da1 * np.where(z1 >= 0, 1.0, 0.1)
        dW1, dB1 = conv2d_dw(x, dz1, W1.shape, 2, 1, 2), dz1.sum((0, 2, 3))
        W1, W2, B1, B2 = W1 - 1e-2 * dW1, W2 - 1e-2 * dW2, B1 - 1e-2 * dB1, B2 - 1e-2 * dB2
        assert abs(losses[-1] - ref_loss) <= 1e-4 * abs(ref_loss)
    assert np.abs(c1.kernel.np() - W1).max() <= 1e-4 * np.abs(W1).max()
    assert np.abs(c2.kernel.np() - W2).max() <= 1e-4 * np.abs(W2).max()
    assert np.abs(c2.bias.np() - B2).max() <= 1e-4 * max(np.abs(B2).max(), 1e-3)
    assert not x_t.has_grad()                          # the input is not trainable: its dX is skipped


@pytest.mark.gpu
def test_encoder_training_step_at_full_channel_widths(nn_hip):
    """The 4-layer encoder of the training-step benchmark at its real widths (3 -> 64 -> 128 -> 256 -> 512, 5x5,
    stride 2, pad 2, leaky_relu(0.1) between layers, loss mean(square), SGD lr 1e-3) on 2 images of 128 x 128: the
    composition the single-layer tests do not see - fused bias / activation epilogues and their backward, strided
    data gradients with all pixel classes in one launch, split-K forward / dgrad on the deep layers, the
    multi-tensor SGD update - against a float64 restatement built from the oracle.  Two steps, so the second runs
    on updated weights.  Loss, every kernel and bias gradient, and every updated kernel within 1e-4 (normalised)."""
    from oracle import conv2d_fwd, conv2d_dx, conv2d_dw
    from tests.gpu_util import say
    nn = nn_hip
    rs = np.random.RandomState(0)
    chans = [3, 64, 128, 256, 512]
    x = rs.uniform(-1, 1, (2, 3, 128, 128)).astype(np.float32)
    ws = [rs.normal(0, np.sqrt(2.0 / (chans[i] * 25)), (chans[i + 1], chans[i], 5, 5)).astype(np.float32) for i in range(4)]
    convs = [nn.Conv2D(chans[i], chans[i + 1], 5, stride=2, padding=2, kernel_initializer=nn.initializer.NumpyArray(ws[i]))
             for i in range(4)]

    class Enc(nn.Module):
        def __init__(self):
            self.convs = convs

        def forward(self, t):
            for i, c in enumerate(self.convs):
                t = c(t)
                if i < 3:
                    t = nn.leaky_relu(t, 0.1)
            return t

    enc = Enc()
    lr = 1e-3
    opt = nn.optimizer.SGD(enc.trainables(), lr=lr)
    x_t = nn.Tensor_from_value(x)
    W = [w.astype(np.float64) for w in ws]
    B = [np.zeros(c) for c in chans[1:]]
    for step in range(2):
        say(f'encoder step {step} at full widths')
        opt.zero_grad()
        loss = nn.square(enc(x_t)).mean()
        loss.backward()
        got_dw = [c.kernel.get_grad().np() for c in convs]
        got_db = [c.bias.get_grad().np() for c in convs]
        opt.step()
        # float64 restatement
        acts, zs = [x.astype(np.float64)], []
        for i in range(4):
            z = conv2d_fwd(acts[-1], W[i], 2, 1, 2) + B[i].reshape(1, -1, 1, 1)
            zs.append(z)
            acts.append(np.where(z >= 0, z, 0.1 * z) if i < 3 else z)
        ref_loss = (zs[3] ** 2).mean()
        assert abs(float(loss.np()[0]) - ref_loss) <= 1e-4 * abs(ref_loss)
        dz = 2 * zs[3] / zs[3].size
        for i in (3, 2, 1, 0):
            dW, dB = conv2d_dw(acts[i], dz, W[i].shape, 2, 1, 2), dz.sum((0, 2, 3))
            assert np.abs(got_dw[i] - dW).max() <= 1e-4 * np.abs(dW).max(), ('dW', step, i)
            assert np.abs(got_db[i].reshape(-1) - dB).max() <= 1e-4 * np.abs(dB).max(), ('dB', step, i)
            if i > 0:
                dz = conv2d_dx(dz, W[i], acts[i].shape, 2, 1, 2) * np.where(zs[i - 1] >= 0, 1.0, 0.1)
            W[i], B[i] = W[i] - lr * dW, B[i] - lr * dB
        for i in range(4):
            assert np.abs(convs[i].kernel.np() - W[i]).max() <= 1e-4 * np.abs(W[i]).max(), ('W', step, i)
            # the update itself, not hidden under the weights' magnitude: v_new - v_old = -lr * g to fp32 rounding of v
            assert np.abs(convs[i].bias.np().reshape(-1) - B[i]).max() <= 1e-4 * max(np.abs(B[i]).max(), 1e-12), ('b', step, i)
    assert not x_t.has_grad()


def test_unfold2d_operator(nn_backend):
    nn = nn_backend
    import litenn_amd.core as nc
    from oracle import unfold_index_map, apply_index_map
    x = np.arange(1, 2 * 3 * 6 * 6 + 1, dtype=np.float32).reshape(2, 3, 6, 6)
    ci = info_conv2d(6, 6, 3, 3, 2, 1, 'same')
    t = nc.op.unfold2D(nn.Tensor_from_value(x), 2, 3, 6, 6, ci.OH, ci.OW, 3, 3, ci.PADL, ci.PADT, 1, 2, 'CJI_NHW', False)
    shape, m = unfold_index_map(2, 3, 6, 6, ci.OH, ci.OW, 3, 3, ci.PADL, ci.PADT, 1, 2, 'CJI_NHW')
    assert t.shape == shape and np.array_equal(t.np(), apply_index_map(x, shape, m))
    with pytest.raises(ValueError):
        nc.op.unfold2D(nn.Tensor_from_value(x), 2, 3, 6, 6, 3, 3, 3, 3, 1, 1, 1, 2, 'N_C_H_W_JI', False)
