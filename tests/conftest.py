import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def cm():
    """The matrix backend, initialised once per session (GPU tests only)."""
    from deepnet_amd import cudamat as cm_
    cm_.cublas_init()
    cm_.CUDAMatrix.init_random(1)
    return cm_


@pytest.fixture(scope="session")
def cc(cm):
    from deepnet_amd import cudamat_conv as cc_
    return cc_


@pytest.fixture
def rng():
    return np.random.default_rng(1234)


def f32(a):
    return np.asarray(a, dtype=np.float32, order='F')
