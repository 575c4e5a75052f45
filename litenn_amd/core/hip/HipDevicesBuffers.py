from .devices import devices
from .HipBuffer import HipBuffer


class HipDevicesBuffers:
    """One lazily allocated HipBuffer per current device
    (counterpart of CLDevicesBuffers.py:4-23); base class of Tensor."""

    def __init__(self, size, init_func=None):
        self._buffers = [HipBuffer(device, size, init_func) for device in devices.get_current()]

    def _get_buffers(self):
        return self._buffers
