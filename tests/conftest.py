import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import th_oracle
    th_oracle.lib()
    return th_oracle


@pytest.fixture(scope="session")
def thc():
    """The engine, initialised on the GPU. Fails loudly if libTHC.so is missing."""
    import cutorch_amd
    cutorch_amd.state()
    return cutorch_amd
