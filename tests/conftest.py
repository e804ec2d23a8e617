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
    from oracle import load_oracle
    return load_oracle()


@pytest.fixture(scope="session")
def hip():
    """The engine binding; GPU tests fail (not skip) if the library is missing."""
    from h2o4gpu_amd.libs import kmeans_hip
    kmeans_hip.lib()
    return kmeans_hip


_FULL_DATA = {}


@pytest.fixture(scope="session")
def full_data():
    """full_data(name, dtype) -> (X, k, iterations) of a benchmark shape at its full size,
    generated once per session (the five shapes take 1.5 minutes to draw; both full-size test
    files use them). About 11 GB of host memory when every shape has been asked for."""
    import numpy as np
    from h2o4gpu_amd import datasets

    def get(name, dtype):
        key = (name, np.dtype(dtype).name)
        if key not in _FULL_DATA:
            X, k, iters = datasets.make(name, 1.0, dtype)
            X.setflags(write=False)
            _FULL_DATA[key] = (X, k, iters)
        return _FULL_DATA[key]
    return get
