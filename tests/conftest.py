import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_backend():
    from oracle.oracle import OracleBackend
    return OracleBackend()


@pytest.fixture(scope="session")
def hip_backend():
    # No fallback: a missing library or device is an error, not a skip.
    from dlf_amd.hip_backend import HipBackend
    return HipBackend("cuda:0")
