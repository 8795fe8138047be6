import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def cuda_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture
def lib_option():
    """Sets experiment switches of the library for one test and restores the library's own choice afterwards."""
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    touched = []

    def setter(name, value):
        hip.set_option(name, value)
        touched.append(name)

    yield setter
    for name in touched:
        hip.set_option(name, -1)
