import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP library through the C ABI)")


@pytest.fixture(scope="session")
def cpu():
    from oracle.cpu_backend import CpuBackend
    return CpuBackend()


@pytest.fixture(scope="session")
def hip():
    # No fallback: a missing library or device is an error, not a skip.
    from forja_amd.hip_backend import HipBackend
    backend = HipBackend(0)
    yield backend
    backend.close()
