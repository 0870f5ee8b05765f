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
    from oracle import tt_oracle

    tt_oracle.lib("fma")  # builds on first use if the shared objects are missing
    return tt_oracle


@pytest.fixture(scope="session")
def tt():
    """The product package; importing it fails loudly when libttamd.so has not been built."""
    import tinytensor_amd

    return tinytensor_amd
