from . import api
from .ShallowMode import ShallowMode
from .HipDevice import HipDevice
from .HipBuffer import HipBuffer
from .devices import devices
from .HipDevicesBuffers import HipDevicesBuffers


def launch(fn, *args):
    """Run `fn(device_index, *per_device_args)` on every current device, taking
    from each HipDevicesBuffers argument that device's pointer (the fan-out of
    CLKernel.run, CLKernel.py:58-62).  A (tensor, 'w') tuple marks an output
    that will be completely overwritten, so its initialiser is skipped.
    Nothing runs in shallow mode.

    The library allocates on its own for some calls (scratch for partial sums, gather tables); when that runs
    out of device memory, blocks idling in the device's pool are released, largest first, and the call is made
    again: the same eviction every tensor allocation gets (CLDevice.py:134-164).  The library allocates before
    it launches anything that writes an output, so a call that failed this way can be repeated."""
    if ShallowMode.active():
        return
    for i, device in enumerate(devices.get_current()):
        resolved = []
        for a in args:
            if isinstance(a, tuple) and len(a) == 2 and a[1] == 'w' and isinstance(a[0], HipDevicesBuffers):
                resolved.append(a[0]._get_buffers()[i].get_ptr(skip_init=True))
            elif isinstance(a, HipDevicesBuffers):
                resolved.append(a._get_buffers()[i].get_ptr())
            else:
                resolved.append(a)
        while True:
            try:
                fn(device.index, *resolved)
                break
            except api.HipException as e:
                if e.code != api.ERR_OOM or not device._release_largest_pooled():
                    raise
