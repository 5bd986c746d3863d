import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run through the C ABI of libmaidenx_hip.so)")


@pytest.fixture(scope="session")
def oracle():
    from helpers import Runner
    return Runner("oracle")


@pytest.fixture(scope="session")
def hip():
    from helpers import Runner
    import maidenx_amd.lib as L
    if L.device_count() < 1:
        pytest.fail("no HIP device visible: GPU tests must run on the MI355X box")
    return Runner("hip")


@pytest.fixture(scope="session")
def mx_oracle():
    from helpers import oracle_host
    return oracle_host()


@pytest.fixture(scope="session")
def mx_hip():
    import maidenx_amd.lib as L
    from maidenx_amd.tensor import host
    if L.device_count() < 1:
        pytest.fail("no HIP device visible: GPU tests must run on the MI355X box")
    return host()
