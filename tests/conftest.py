import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pa():
    """The product package; GPU tests fail (not skip) when the HIP library is missing."""
    import ai_infra_train_infer_amd as pkg
    return pkg


@pytest.fixture(scope="session")
def lib(pa):
    return pa._native.load()


@pytest.fixture(scope="session")
def gpu():
    import torch
    assert torch.cuda.is_available(), "GPU test run on a machine without a GPU"
    return torch.device("cuda:0")
