import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


@pytest.fixture(scope="session")
def queue():
    """One HIP stream for the whole session (the reference's `ctx` fixture, conftest.py:5-7)."""
    from nengo_ocl_amd.hipraggedarray import Queue

    return Queue(0)


@pytest.fixture
def rng():
    return np.random.RandomState(20240607)
