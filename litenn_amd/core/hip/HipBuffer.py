import numpy as np

from . import api
from .ShallowMode import ShallowMode


class HipBuffer:
    """Lazily allocated block of device memory (counterpart of CLBuffer,
    CLBuffer.py:5-123).  The device pointer is obtained from the device's pool
    on first use; `init_func(buffer)` then fills it.

     size        bytes
     init_func   callable(HipBuffer) run right after physical allocation
    """
    __slots__ = ['device', 'size', 'init_func', '_ptr', '_version', '_derived', '__weakref__']
    _object_count = 0

    def __init__(self, device, size, init_func=None):
        HipBuffer._object_count += 1
        self._ptr = None
        self._version = 0      # grows whenever the contents may have changed (any access that is not read-only)
        self._derived = None   # {key: (version, HipBuffer)}: copies in another layout, valid for that version only
        if size <= 0:
            raise ValueError(f'Create HipBuffer with {size} size.')
        self.device = device
        self.size = size
        self.init_func = init_func

    def __del__(self):
        HipBuffer._object_count -= 1
        self.free_ptr()

    def has_ptr(self):
        return self._ptr is not None

    def get_ptr(self, skip_init=False, readonly=False):
        """Device address.  skip_init=True is for a caller about to overwrite
        every element: the initialiser is not run on first allocation.
        readonly=True is a promise not to write through the pointer; every other access counts as a change of
        the contents and invalidates copies derived from them (see derived())."""
        if self._ptr is None:
            self._ptr = self.device._mem_alloc(self.size)
            if self.init_func is not None and not skip_init:
                self.init_func(self)
        if not readonly:
            self._version += 1
        return self._ptr

    def derived(self, key, size, make):
        """A buffer computed from this one's current contents (the weights in a kernel's own layout), kept until
        the contents change: make(src_ptr, dst_ptr) fills it.  Returns the derived HipBuffer."""
        src = self.get_ptr(readonly=True)
        if self._derived is None:
            self._derived = {}
        entry = self._derived.get(key)
        if entry is not None and entry[0] == self._version:
            return entry[1]
        buf = entry[1] if entry is not None else HipBuffer(self.device, size)
        make(src, buf.get_ptr(skip_init=True))
        self._derived[key] = (self._version, buf)
        return buf

    def free_ptr(self):
        self._derived = None
        if self._ptr is not None:
            self.device._mem_free(self._ptr, self.size)
            self._ptr = None

    def set(self, value):
        """Copy from another HipBuffer (same size) or from an np.ndarray whose
        nbytes equal the buffer size; an upload returns once the host array
        may be reused (CLBuffer.py:50-80)."""
        if isinstance(value, HipBuffer):
            if value is self:
                return
            if self.size != value.size:
                raise Exception(f'Unable to copy from HipBuffer with {value.size} size to buffer with {self.size} size.')
            if ShallowMode.active():
                return
            if self.device is value.device:
                api.memcpy_d2d(self.device.index, self.get_ptr(skip_init=True), value.get_ptr(readonly=True), self.size)
            else:
                self.set(value.np())
            return
        if not isinstance(value, np.ndarray):
            raise ValueError(f'Invalid type {value.__class__}. Must be np.ndarray.')
        if value.nbytes != self.size:
            raise ValueError(f'Value size {value.nbytes} does not match HipBuffer size {self.size}.')
        if ShallowMode.active():
            return
        api.memcpy_h2d(self.device.index, self.get_ptr(skip_init=True), np.ascontiguousarray(value))

    _allowed_fill_types = (np.float32, np.int32, np.uint32)

    def fill(self, value):
        """Fill the whole buffer with one 32-bit scalar (CLBuffer.py:83-96)."""
        if isinstance(value, (np.float64, np.float16)):
            value = np.float32(value)
        if not isinstance(value, HipBuffer._allowed_fill_types):
            raise ValueError(f'Unknown type {value.__class__}. Allowed types : {HipBuffer._allowed_fill_types} ')
        if ShallowMode.active():
            return
        api.fill_u32(self.device.index, self.get_ptr(skip_init=True), int(value.view(np.uint32)), self.size // 4)

    def np(self, shape=None, dtype=np.float32):
        """Download as np.ndarray (CLBuffer.py:99-115); blocks until the data
        has arrived."""
        if dtype is not np.float32 and np.dtype(dtype) != np.float32:
            raise ValueError('only float32 buffers exist')
        if shape is None or len(shape) == 0:
            shape = (self.size // 4,)
        out = np.empty(tuple(shape), np.float32)
        if out.nbytes != self.size:
            raise ValueError(f'Unable to represent HipBuffer with size {self.size} as shape {shape} with dtype {dtype}')
        if not ShallowMode.active():
            api.memcpy_d2h(self.device.index, out, self.get_ptr(readonly=True))
        return out

    def __str__(self):
        return f'HipBuffer [{self.size} bytes] on {self.device}'

    __repr__ = __str__
