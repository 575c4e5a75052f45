"""Helpers for the GPU parity tests: raw device arrays over the C ABI."""
import sys

import numpy as np


def say(msg):
    """Name the case before it touches the GPU, flushed, so a lost box still tells which one ran."""
    print(msg, flush=True)
    sys.stdout.flush()


class DevArr:
    """A device allocation holding a float32 array (uploaded on construction)."""

    def __init__(self, api, array=None, shape=None, dev=0, fill=None):
        self.api, self.dev = api, dev
        if array is not None:
            array = np.ascontiguousarray(array, dtype=np.float32)
            shape = array.shape
        self.shape = tuple(shape)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * 4
        self.ptr = api.malloc(dev, max(self.nbytes, 4))
        if array is not None:
            api.memcpy_h2d(dev, self.ptr, array)
        elif fill is not None:
            api.fill_f32(dev, self.ptr, fill, self.nbytes // 4)

    def get(self):
        out = np.empty(self.shape, np.float32)
        self.api.memcpy_d2h(self.dev, out, self.ptr)
        return out

    def free(self):
        if self.ptr:
            self.api.free(self.dev, self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def rel_err(got, ref):
    """max |got - ref| / max |ref|: the normalised error the parity bar is stated in."""
    ref = np.asarray(ref, np.float64)
    denom = np.abs(ref).max()
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / (denom if denom > 0 else 1.0))
