import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


@pytest.fixture(scope='session')
def hip():
    """The loaded C-ABI library bound to device 0 (GPU tests only)."""
    from litenn_amd.core.hip import api
    if api.device_count() < 1:
        pytest.fail('no HIP device visible: GPU tests must run on a GPU box')
    return api


def _reset_registry():
    import gc
    import litenn_amd as nn
    from litenn_amd.core.hip import devices
    gc.collect()
    try:
        nn.cleanup()
    finally:
        devices._current_devices = None
        devices._all_devices = None


@pytest.fixture(params=[pytest.param('fake'), pytest.param('hip', marks=pytest.mark.gpu)])
def nn_backend(request, monkeypatch, capsys):
    """`import litenn_amd as nn` bound either to the numpy stand-in (host
    logic, runs anywhere) or to the real library on GPU 0."""
    import litenn_amd as nn
    from litenn_amd.core.hip import devices
    devices._current_devices = None
    devices._all_devices = None
    fake = None
    if request.param == 'fake':
        from tests import fake_hip
        fake = fake_hip.install(monkeypatch)
    nn._test_fake = fake
    yield nn
    nn._test_fake = None
    _reset_registry()


@pytest.fixture
def nn_hip(capsys):
    """`import litenn_amd as nn` on the real library and GPU 0 only (for cases too large for the numpy stand-in)."""
    import litenn_amd as nn
    from litenn_amd.core.hip import devices
    devices._current_devices = None
    devices._all_devices = None
    nn._test_fake = None
    yield nn
    _reset_registry()
