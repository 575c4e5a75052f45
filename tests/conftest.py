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
