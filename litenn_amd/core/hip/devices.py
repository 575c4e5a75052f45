from collections.abc import Iterable
from typing import List

from . import api
from .HipBuffer import HipBuffer
from .HipDevice import HipDevice
from .ShallowMode import ShallowMode


class devices:
    """Static registry of the current device(s) (counterpart of devices.py:8-170;
    the interactive chooser of devices.py:173-261 is not carried over)."""

    _current_devices = None
    _all_devices = None

    @staticmethod
    def _shallow_mode():
        """`with devices._shallow_mode():` runs ops without touching the GPU."""
        return ShallowMode()

    @staticmethod
    def get_all() -> List[HipDevice]:
        if devices._all_devices is None:
            found = []
            for i in range(api.device_count()):
                info = api.device_info(i)
                found.append(HipDevice(i, info['name'], info['total_mem'], info['compute_units']))
            devices._all_devices = found
        return devices._all_devices

    @staticmethod
    def get_by_idx(index):
        for dev in devices.get_all():
            if dev.index == index:
                return dev
        return None

    @staticmethod
    def get_best():
        """The device with the most memory (devices.py:145-156)."""
        best = None
        for dev in devices.get_all():
            if best is None or dev.global_mem_size > best.global_mem_size:
                best = dev
        return best

    @staticmethod
    def get_equal(device):
        return [d for d in devices.get_all() if d.name == device.name]

    @staticmethod
    def get_current() -> List[HipDevice]:
        if devices._current_devices is None:
            best = devices.get_best()
            if best is None:
                raise Exception('No HIP device found: this package runs on AMD MI355X only.')
            devices.set_current(best)
        return devices._current_devices

    @staticmethod
    def set_current(device_or_list):
        if HipBuffer._object_count != 0:
            raise Exception('You cannot set current devices while any HipBuffer objects exists.')
        devices.cleanup()
        if isinstance(device_or_list, Iterable):
            device_or_list = tuple(device_or_list)
        else:
            device_or_list = (device_or_list,)
        if len(device_or_list) == 0:
            raise ValueError('device_or_list cannot be empty')
        for d in device_or_list:
            if not isinstance(d, HipDevice):
                raise ValueError(f'argument {d.__class__} should be HipDevice')
        print(f'Using {", ".join(d.name for d in device_or_list)}')
        devices._current_devices = device_or_list

    @staticmethod
    def cleanup():
        if HipBuffer._object_count != 0:
            raise Exception(f'Unable to cleanup while {HipBuffer._object_count} HipBuffer objects exist.')
        if devices._current_devices is not None:
            for d in devices._current_devices:
                d._cleanup()

    @staticmethod
    def wait():
        for d in devices.get_current():
            d.wait()
