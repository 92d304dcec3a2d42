import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu and needs a GPU: none is visible")
    return torch.device("cuda:0")


@pytest.fixture
def tuning():
    """Sets library tuning switches for one test and puts the old values back afterwards:
    tuning("decode_flat", 1)."""
    from aici_amd import kernels as K

    saved = {}

    def set_switch(name, value):
        if name not in saved:
            saved[name] = K.tuning_get(name)
        K.tuning_set(name, value)

    yield set_switch
    for name, value in saved.items():
        K.tuning_set(name, value)
