"""The C-ABI library loads without a GPU and exports exactly what
include/litenn_hip.h declares; the ctypes binding covers every symbol."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, 'include', 'litenn_hip.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(lnn_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
    from litenn_amd.core.hip import api
    names = _declared()
    assert len(names) >= 25 and 'lnn_conv2d_fwd_f32' in names and 'lnn_gemm_f32' in names
    lib = ctypes.CDLL(api.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f'{n} is declared in the header but not exported'


def test_binding_covers_the_header():
    from litenn_amd.core.hip import api
    bound = set(api.SIGNATURES) | {'lnn_last_error'}
    assert bound == set(_declared())


def test_no_device_is_reported_not_faked():
    """Without a GPU the library reports zero devices and every device call
    fails with NO_DEVICE; nothing falls back to the host."""
    from litenn_amd.core.hip import api
    if api.device_count() > 0:
        return
    import pytest
    with pytest.raises(api.HipException) as e:
        api.malloc(0, 1024)
    assert e.value.code == api.ERR_NO_DEVICE
    import litenn_amd as nn
    from litenn_amd.core.hip import devices
    devices._all_devices = devices._current_devices = None
    with pytest.raises(Exception, match='No HIP device'):
        nn.Tensor((4,))
    devices._all_devices = devices._current_devices = None


def test_desc_struct_layout_matches_header():
    from litenn_amd.core.hip import api
    assert ctypes.sizeof(api.ConvDesc) == 13 * 4
    assert [f[0] for f in api.ConvDesc._fields_] == ['N', 'C', 'IH', 'IW', 'O', 'KH', 'KW', 'OH', 'OW', 'PADL',
                                                     'PADT', 'stride', 'dilation']
