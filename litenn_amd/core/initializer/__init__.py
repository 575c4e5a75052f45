"""Initializers (nn.initializer.*).

Scalar and NumpyArray are the ones the conv2D / matmul path needs
(initializer/Scalar.py:5-20, NumpyArray.py:5-21).  The random initialisers
fill the buffer on the device from a counter hash, as the reference's do
(initializer/RandomUniform.py:13-27, RandomNormal.py:10-30): the host only
draws the 31-bit seed from numpy's global generator, so np.random.seed(k)
fixes the initial weights here exactly as it does there.
"""
import numpy as np

import litenn_amd.core as nc
from litenn_amd.core.hip import api
from litenn_amd.core.hip.ShallowMode import ShallowMode


class Initializer:
    """Base class.  Subclasses implement initialize_CLBuffer(buffer, shape):
    fill the freshly allocated device buffer (buffer.fill / buffer.set).
    The method keeps the reference's name so initialisers written against
    initializer/Initializer.py:29-36 work unchanged."""

    def has_fan_in(self): return False
    def has_fan_out(self): return False

    def initialize_CLBuffer(self, buffer, tensor_shape):
        raise NotImplementedError()

    def __str__(self): return 'Initializer'
    def __repr__(self): return self.__str__()


class _ScalarInit(Initializer):
    def __init__(self, value):
        self.value = value

    def initialize_CLBuffer(self, buffer, tensor_shape):
        buffer.fill(np.float32(self.value))

    def __str__(self): return f'Scalar ({self.value})'


def Scalar(value):
    """Every element = value."""
    return nc.Cacheton.get(_ScalarInit, value)


class _NumpyArrayInit(Initializer):
    def __init__(self, np_array):
        self.np_array = np.ascontiguousarray(np_array, dtype=np.float32).copy()

    def initialize_CLBuffer(self, buffer, tensor_shape):
        buffer.set(self.np_array)

    def __str__(self): return f'NumpyArray {self.np_array.shape}'


def NumpyArray(np_array):
    """Upload a copy of np_array (converted to float32)."""
    return _NumpyArrayInit(np_array)


def _draw_seed():
    """The reference's seed draw (RandomUniform.py:26, RandomNormal.py:29)."""
    return int(np.random.randint(2147483648))


class _RandomUniform(Initializer):
    def __init__(self, low=0.0, high=1.0):
        self.low, self.high = low, high

    def initialize_CLBuffer(self, buffer, tensor_shape):
        seed = _draw_seed()
        if ShallowMode.active():
            return
        api.random_uniform(buffer.device.index, buffer.get_ptr(skip_init=True), buffer.size // 4, seed,
                           self.low, self.high)

    def __str__(self): return f'RandomUniform low={self.low}, high={self.high}'


def RandomUniform(low=0.0, high=1.0):
    """U[low, high] from the device hash (RandomUniform.py:32-43)."""
    return nc.Cacheton.get(_RandomUniform, low, high)


class _RandomNormal(Initializer):
    def __init__(self, mean=0.0, stddev=1.0):
        self.mean, self.stddev = mean, stddev

    def initialize_CLBuffer(self, buffer, tensor_shape):
        seed = _draw_seed()
        if ShallowMode.active():
            return
        api.random_normal(buffer.device.index, buffer.get_ptr(skip_init=True), buffer.size // 4, seed,
                          self.mean, self.stddev)

    def __str__(self): return f'RandomNormal mean={self.mean}, stddev={self.stddev}'


def RandomNormal(mean=0.0, stddev=1.0):
    """N(mean, stddev) by Box-Muller on the device hash (RandomNormal.py:35-46)."""
    return nc.Cacheton.get(_RandomNormal, mean, stddev)


class _FanInit(Initializer):
    """He / Glorot: a RandomUniform(-a, a) with a = sqrt(3)*std or a RandomNormal(0, std), chosen on first use
    once the layer has supplied the fans (He.py:18-33, Glorot.py:20-35).

    Every call of HeNormal() etc. returns a fresh object, so each layer that fills in fan_in / fan_out gets its
    own bound; the reference hands out one cached object per argument tuple, which keeps the fans (and the
    bound) of the first layer that used it."""

    def __init__(self, type, gain, fan_in=None, fan_out=None):
        self.type, self.gain, self.fan_in, self.fan_out = type, gain, fan_in, fan_out
        self.initer = None

    def has_fan_in(self): return True

    def _std(self):
        raise NotImplementedError()

    def initialize_CLBuffer(self, buffer, tensor_shape):
        if self.initer is None:
            std = self._std()
            if self.type == 'uniform':
                a = np.sqrt(3.0) * std
                self.initer = RandomUniform(-a, a)
            else:
                self.initer = RandomNormal(0.0, std)
        self.initer.initialize_CLBuffer(buffer, tensor_shape)


class _InitHe(_FanInit):
    def _std(self):
        if self.fan_in is None:
            raise ValueError(f'fan_in should be set for {str(self)}')
        return self.gain * np.sqrt(2.0 / self.fan_in)

    def __str__(self): return f'InitHe type={self.type}, gain={self.gain}, fan_in={self.fan_in}'


class _InitGlorot(_FanInit):
    def has_fan_out(self): return True

    def _std(self):
        if self.fan_in is None or self.fan_out is None:
            raise ValueError(f'fan_in/fan_out should be set for {str(self)}')
        return self.gain * np.sqrt(2.0 / (self.fan_in + self.fan_out))

    def __str__(self):
        return f'InitGlorot type={self.type}, gain={self.gain}, fan_in={self.fan_in}, fan_out={self.fan_out}'


def HeUniform(gain=2.0, fan_in=None):
    """U(-a, a), a = sqrt(3)*gain*sqrt(2/fan_in); default gain 2 (He.py:36-49)."""
    return _InitHe('uniform', gain, fan_in)


def HeNormal(gain=1.0, fan_in=None):
    """N(0, gain*sqrt(2/fan_in)) (He.py:51-64)."""
    return _InitHe('normal', gain, fan_in)


def GlorotUniform(gain=1.0, fan_in=None, fan_out=None):
    """U(-a, a), a = sqrt(3)*gain*sqrt(2/(fan_in+fan_out)) (Glorot.py:37-59)."""
    return _InitGlorot('uniform', gain, fan_in, fan_out)


def GlorotNormal(gain=1.0, fan_in=None, fan_out=None):
    """N(0, gain*sqrt(2/(fan_in+fan_out))) (Glorot.py:61-78)."""
    return _InitGlorot('normal', gain, fan_in, fan_out)
