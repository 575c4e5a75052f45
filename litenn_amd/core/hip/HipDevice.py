from . import api
from .ShallowMode import ShallowMode


class HipDevice:
    """One MI355X as seen by the tensor layer.

    Counterpart of CLDevice (CLDevice.py:6-194) with the OpenCL context, queue
    and JIT kernel cache gone: kernels are prebuilt in the library and run on
    the library's per-device stream.  What stays is the exact-size-keyed pool
    of device allocations with largest-first eviction on out-of-memory
    (CLDevice.py:120-178) and the memory counters (CLDevice.py:39-49).

    properties: .index .name .global_mem_size .is_cpu .compute_units
    """

    def __init__(self, index, name, global_mem_size, compute_units):
        self.index = index
        self.name = name
        self.global_mem_size = global_mem_size
        self.compute_units = compute_units
        self.is_cpu = False
        self._pool = {}
        self._total_buffers_allocated = 0
        self._total_buffers_pooled = 0
        self._total_memory_allocated = 0
        self._total_memory_pooled = 0

    def get_used_memory(self):
        return self.get_total_allocated_memory() - self.get_total_pooled_memory()

    def get_total_allocated_memory(self):
        return self._total_memory_allocated

    def get_total_pooled_memory(self):
        return self._total_memory_pooled

    def wait(self):
        """Block until everything queued on this device has finished."""
        api.synchronize(self.index)

    # ---- internal ---------------------------------------------------------
    def _mem_alloc(self, size):
        """Device pointer of `size` bytes: reuse a pooled block of exactly
        that size, else allocate; on out-of-memory release pooled blocks,
        largest first, and retry (CLDevice.py:134-164)."""
        if ShallowMode.active():
            raise Exception('Memory allocation is not allowed in shallow mode.')
        stack = self._pool.get(size)
        if stack:
            ptr = stack.pop()
            self._total_memory_pooled -= size
            self._total_buffers_pooled -= 1
            return ptr
        while True:
            try:
                ptr = api.malloc(self.index, size)
            except api.HipException as e:
                if e.code == api.ERR_OOM and self._release_largest_pooled():
                    continue
                raise Exception(f'Unable to allocate {size // 1024**2}Mb on {self}. additional_log: {e}')
            self._total_buffers_allocated += 1
            self._total_memory_allocated += size
            return ptr

    def _release_largest_pooled(self):
        for key in sorted(self._pool, reverse=True):
            stack = self._pool[key]
            if stack:
                api.free(self.index, stack.pop())
                self._total_buffers_pooled -= 1
                self._total_buffers_allocated -= 1
                self._total_memory_pooled -= key
                self._total_memory_allocated -= key
                return True
        return False

    def _mem_free(self, ptr, size):
        """Return a block to the pool (CLDevice.py:167-178).  Work already
        queued on the stream that uses the block finishes before any later
        launch that reuses it, because the stream is in order."""
        self._pool.setdefault(size, []).append(ptr)
        self._total_memory_pooled += size
        self._total_buffers_pooled += 1

    def _cleanup(self):
        """Free every pooled block and the library's per-device state."""
        if self._total_buffers_pooled != self._total_buffers_allocated:
            raise Exception('Unable to cleanup HipDevice, while not all buffers are pooled/deallocated.')
        while self._release_largest_pooled():
            pass
        self._pool = {}
        api.release_device(self.index)

    def __str__(self):
        return f'[{self.index}]:[{self.name}][{self.global_mem_size / 1024**3 :.3} GB]'

    __repr__ = __str__
