import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle

    _oracle.build()
    return _oracle


@pytest.fixture(scope="session")
def hip():
    """(device, pool) on GPU 0 through the C ABI. No fallback: a missing library or GPU fails the test."""
    import zyx_amd

    pools, devices = zyx_amd.initialize_device(zyx_amd.HIPConfig(device_ids=[0]))
    yield devices[0], pools[0]
    pools[0].deinitialize()
