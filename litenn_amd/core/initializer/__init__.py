"""Initializers (nn.initializer.*).

Scalar and NumpyArray are the ones the conv2D / matmul path needs
(initializer/Scalar.py:5-20, NumpyArray.py:5-21).  The random initialisers
draw on the HOST with numpy and upload the result; the reference instead runs
a hash-based generator on the device (initializer/RandomNormal.py:6-30), whose
stream is not reproduced here.
"""
import math

import numpy as np

import litenn_amd.core as nc


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


class _HostRandom(Initializer):
    def _draw(self, shape):
        raise NotImplementedError()

    def initialize_CLBuffer(self, buffer, tensor_shape):
        buffer.set(np.ascontiguousarray(self._draw(tuple(tensor_shape)), dtype=np.float32))


class RandomUniform(_HostRandom):
    def __init__(self, low=-1.0, high=1.0):
        self.low, self.high = low, high

    def _draw(self, shape): return np.random.uniform(self.low, self.high, shape)
    def __str__(self): return f'RandomUniform low={self.low}, high={self.high}'


class RandomNormal(_HostRandom):
    def __init__(self, mean=0.0, stddev=1.0):
        self.mean, self.stddev = mean, stddev

    def _draw(self, shape): return np.random.normal(self.mean, self.stddev, shape)
    def __str__(self): return f'RandomNormal mean={self.mean}, stddev={self.stddev}'


class _FanInit(_HostRandom):
    def __init__(self, gain=1.0, fan_in=None, fan_out=None):
        self.gain, self.fan_in, self.fan_out = gain, fan_in, fan_out

    def has_fan_in(self): return True


class HeNormal(_FanInit):
    """N(0, gain*sqrt(2/fan_in))  (He.py:18-33,51-64)."""
    def __init__(self, gain=1.0, fan_in=None):
        super().__init__(gain, fan_in)

    def _draw(self, shape):
        return np.random.normal(0.0, self.gain * math.sqrt(2.0 / self.fan_in), shape)


class HeUniform(_FanInit):
    """U(-l, l), l = gain*sqrt(6/fan_in); default gain 2  (He.py:18-49)."""
    def __init__(self, gain=2.0, fan_in=None):
        super().__init__(gain, fan_in)

    def _draw(self, shape):
        lim = self.gain * math.sqrt(6.0 / self.fan_in)
        return np.random.uniform(-lim, lim, shape)


class GlorotNormal(_FanInit):
    """N(0, gain*sqrt(2/(fan_in+fan_out)))  (Glorot.py:20-35,61-78)."""
    def has_fan_out(self): return True

    def _draw(self, shape):
        return np.random.normal(0.0, self.gain * math.sqrt(2.0 / (self.fan_in + self.fan_out)), shape)


class GlorotUniform(_FanInit):
    """U(-l, l), l = gain*sqrt(6/(fan_in+fan_out))  (Glorot.py:20-35,37-59)."""
    def has_fan_out(self): return True

    def _draw(self, shape):
        lim = self.gain * math.sqrt(6.0 / (self.fan_in + self.fan_out))
        return np.random.uniform(-lim, lim, shape)
