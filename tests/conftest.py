import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 device (run on the GPU box)")


@pytest.fixture(scope="session")
def O():
    import oracle
    return oracle


@pytest.fixture(scope="session")
def tfq():
    return importlib.import_module("transformers-fusion_amd")


@pytest.fixture(scope="session")
def gpu(tfq):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    tfq.init(0)
    return torch.device("cuda:0")
