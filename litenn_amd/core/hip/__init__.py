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
    that will be completely overwritten, so its initialiser is skipped; a
    (tensor, 'r') tuple one that is only read (a plain tensor argument counts
    as possibly written, which invalidates layout copies derived from it).
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
            elif isinstance(a, tuple) and len(a) == 2 and a[1] == 'r' and isinstance(a[0], HipDevicesBuffers):
                resolved.append(a[0]._get_buffers()[i].get_ptr(readonly=True))
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


def cached_permuted_copies(tensors):
    """For an optimizer step over `tensors`: per tensor None, or (key, copies, C, KH*KW, layout) when every device
    buffer of the tensor holds exactly one permuted copy Wp[o][tap][c] (permuted_weights below; layout = how the
    tensor itself is stored, W_OIHW or W_IOHW) - the update kernels can then store the new values in the copy too.
    copies is a launch() argument."""
    out = []
    for t in tensors:
        key, copies = None, []
        for buf in t._get_buffers():
            keys = [k for k in (buf._derived or {}) if k[0] == 'wp']
            if len(keys) != 1 or (key is not None and keys[0] != key):
                key = None
                break
            key = keys[0]
            copies.append(buf._derived[key][1])
        if key is None or key[2] * key[3] * key[4] * key[5] != t.shape.size:
            out.append(None)
        else:
            out.append((key, _BufferList(copies), key[3], key[4] * key[5], key[1]))
    return out


def keep_permuted_copies(tensors, cached):
    """After an update that wrote the copies of cached_permuted_copies(): they are valid for the tensors' new contents."""
    if ShallowMode.active():
        return
    for t, c in zip(tensors, cached):
        if c is not None:
            for buf, copy in zip(t._get_buffers(), c[1]._get_buffers()):
                buf._derived[c[0]] = (buf._version, copy)


class _BufferList(HipDevicesBuffers):
    """Per-device buffers that already exist, in the shape launch() takes."""

    def __init__(self, buffers):
        self._buffers = buffers


def permuted_weights(kernel_t, desc, w_layout=api.W_OIHW):
    """The convolution weights of kernel_t in the layout the tap-major kernels read, Wp[o][tap][c], as a launch()
    argument (pass it as (result, 'r')).  One copy per device, made on first use and again only after kernel_t's
    contents may have changed (an optimizer step, set(), fill(), any launch that took it as a plain argument):
    forward and data gradient of a training step, and every pass of an inference loop, share it.
    w_layout W_IOHW: kernel_t is stored (C, O, KH, KW) relative to desc, as a transposed convolution keeps it.
    A 1x1 kernel stored OIHW already has the layout and is returned itself."""
    if w_layout == api.W_OIHW and desc.KH * desc.KW == 1:
        return kernel_t
    if ShallowMode.active():
        return kernel_t
    key = ('wp', int(w_layout), desc.O, desc.C, desc.KH, desc.KW)
    size = desc.O * desc.C * desc.KH * desc.KW * 4
    out = []
    for buf in kernel_t._get_buffers():
        dev = buf.device.index
        out.append(buf.derived(key, size, lambda src, dst, dev=dev: api.conv2d_permute_weights(dev, desc, src, w_layout, dst)))
    return _BufferList(out)
